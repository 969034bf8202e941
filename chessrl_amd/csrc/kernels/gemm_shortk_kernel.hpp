// C[M,N] = descale * A[M,K] · W[N,K]^T for e4m3 operands with K = 256 (two 128-byte slabs) and a large 16-bit output:
// the shape of the shared attention-bias generator (M = positions x heads, N = 4096). With so short a K a tile of the
// general kernels is all prologue and epilogue (of the 11 us a 256x256 tile lives, 4 are its main loop), and no
// workgroup can overlap them with another's: the product ran at half the rate its 1 GB of output can be written at.
//
// Here a workgroup of eight waves owns 256 rows of A for the whole launch and walks N in steps of 128 columns:
//  * its A operand fragments are loaded once, straight from global memory into registers (64 per lane: the whole K of
//    the wave's 64 rows), and never pass through LDS;
//  * the 128 weight rows of a step (32 KB, both slabs) arrive by direct-to-LDS loads in a two-stage ring, requested
//    one step ahead; one barrier per step;
//  * a step is 16 MFMAs per wave (a 64x64 wave tile, 32x32x64 e4m3) followed by the wave's own epilogue: scale, convert
//    to 16 bits, transpose 32x64 strips through a wave-private LDS patch (16-bit data: half the LDS traffic of the fp32
//    patch of the general epilogue) and store whole 128-byte row segments with the non-temporal hint;
//  * the loop is rotated (write out step - 1, then multiply step), so that the stores of a step drain and the weights
//    of the next one arrive under an MFMA phase before the one wait per step, which has to be for all of them;
//  * optionally (GemmArgs::c_blocked) C is laid out in blocks of 256 rows x 128 columns, so that the 64 KB a workgroup
//    writes per step are consecutive addresses.
// Same K order and the same arithmetic per element as the tiled kernels: bit-equal results.
#pragma once
#include "gemm_dmam_kernel.hpp"

namespace crl {

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

struct ShortKCfg {
  static constexpr int BM = 256, BN = 128, WGM = 4, WGN = 2, NW = 8, NT = 512;
  static constexpr int WM = 64, WN = 64, TM = 2, TN = 2;
  static constexpr int ROWB = 128, NSLAB = 2, KSTEPS = 4;        // K = 256 bytes: four MFMA K steps of 64
  static constexpr int SLAB_BYTES = BN * ROWB;                     // 16 KB: one slab of a step's weight rows
  static constexpr int STAGE_BYTES = NSLAB * SLAB_BYTES;           // 32 KB
  static constexpr int RING_BYTES = 2 * STAGE_BYTES;               // 64 KB
  static constexpr int PATCH_BYTES = 32 * WN * 2;                  // 4 KB: a 32x64 strip of 16-bit values
  static constexpr int LDS_BYTES = RING_BYTES + NW * TM * PATCH_BYTES;   // 128 KB
  static constexpr int LOADS = STAGE_BYTES / 1024 / NW;            // 4 wave-instructions (8 rows of 128 bytes each) per wave and step
};

template <int OUT_DT>
__global__ void __launch_bounds__(ShortKCfg::NT, 2) gemm_shortk_kernel(const GemmArgs a) {
  typedef ShortKCfg Cfg;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, KSTEPS = Cfg::KSTEPS, LOADS = Cfg::LOADS;
  extern __shared__ __align__(16) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % Cfg::WGM, wn = wave / Cfg::WGM;
  const int lr = lane & 31, g = lane >> 5;
  const int m0 = blockIdx.x * Cfg::BM;
  const int nsteps = a.N / Cfg::BN;

  // Weight loads: wave-instruction q = 4 wave + i of a stage's 32 covers rows 8 (q & 15) .. +8 of slab q >> 4, eight
  // 16-byte chunks per row, the swizzle applied on the global side.
  uint32_t voff[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int q = wave * LOADS + i;
    const int row = 8 * (q & 15) + (lane >> 3);
    voff[i] = (uint32_t)row * (uint32_t)a.ldw + (q >> 4) * Cfg::ROWB + (((lane & 7) ^ lds_swizzle(row)) << 4);
  }
  const long wspan = (long)a.N * a.ldw;
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(a.W), 0, (int)(wspan < 0x7fffffffL ? wspan : 0x7fffffffL), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_none = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(a.W), 0, 0, 0x00020000);
  const int step_bytes = Cfg::BN * (int)a.ldw;
  auto issue_step = [&](int step) {
    const __amdgpu_buffer_rsrc_t r = step < nsteps ? rsrc_w : rsrc_none;
    uint8_t* dst = smem + (step & 1) * Cfg::STAGE_BYTES + wave * LOADS * 1024;
    static_for<0, LOADS>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)(dst + i * 1024), 16, (int)voff[i], step * step_bytes, 0, 0);
    });
  };
  issue_step(0);

  // The wave's A fragments: rows m0 + 64 wm + 32 tm + lr, bytes [64 ks + 32 g, +32) of each. Rows past M repeat the last one.
  Frag<DT_FP8> xf[TM][KSTEPS];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    int m = m0 + wm * Cfg::WM + tm * 32 + lr;
    m = m < a.M ? m : a.M - 1;
    const uint8_t* row = reinterpret_cast<const uint8_t*>(a.A) + (long)m * a.lda + 32 * g;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      xf[tm][ks].lo = *reinterpret_cast<const i32x4_t*>(row + 64 * ks);
      xf[tm][ks].hi = *reinterpret_cast<const i32x4_t*>(row + 64 * ks + 16);
    }
  }

  // Weight fragment addresses: row 64 wn + 32 tn + lr of a slab, chunk (4 (ks & 1) + 2 g + half) ^ swizzle(row).
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)smem);
  uint32_t wrow[TN];
  int wsw[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int row = wn * Cfg::WN + tn * 32 + lr;
    wrow[tn] = lds0 + row * Cfg::ROWB;
    wsw[tn] = lds_swizzle(row) ^ (2 * g);
  }
  auto read_w = [&](uint32_t stage_off, int tn, int ks, int half) -> i32x4_t {
    const int c = 4 * (ks & 1) + half;
    return *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>(wrow[tn] + stage_off + (ks >> 1) * Cfg::SLAB_BYTES + ((c ^ wsw[tn]) << 4));
  };

  // Epilogue addressing. Patch (per wave and strip tm): 32 rows of 128 bytes, 16-byte chunk c of row r at chunk position
  // c ^ (r & 7), its two 8-byte halves exchanged in rows with bit 3 set (so that the sixteen lanes of one LDS cycle,
  // rows r and r + 8 among them, hit sixteen different 8-byte slots). A lane writes 8 bytes (4 columns) per MFMA tile
  // and row quad, and reads back chunk ec of rows er + 8 it.
  // The patch is written and read with instructions spelled out: in front of a compiler-generated LDS store the
  // compiler waits for every direct-to-LDS load in flight (it cannot tell that they land elsewhere), i.e. for the
  // weights of the next step, requested a moment ago.
  const uint32_t patch0 = lds0 + Cfg::RING_BYTES + wave * (TM * Cfg::PATCH_BYTES);
  uint32_t pw[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) pw[c] = patch0 + lr * 128 + ((c ^ (lr & 7)) << 4) + ((g ^ ((lr >> 3) & 1)) << 3);
  const int er = lane >> 3, ec = lane & 7;
  const uint32_t pr = patch0 + er * 128 + ((ec ^ er) << 4);
  const float descale = a.descale;
  // Output addressing: a scalar base per step plus one lane offset per (strip, row group). c_blocked: C is stored in
  // blocks of (256 rows) x (128 columns), 64 KB each and contiguous, block (m / 256, n / 128) at index (m / 256) * (N /
  // 128) + n / 128: a workgroup then writes 64 KB of consecutive addresses per step instead of 256 pieces of 256 bytes a
  // row stride apart (measured on M = 131072, N = 4096: 316 -> 216 us with everything else equal).
  const uint32_t row_stride = a.c_blocked ? Cfg::BN * 2 : (uint32_t)a.ldc * 2;
  const long step_stride = a.c_blocked ? (long)Cfg::BM * Cfg::BN * 2 : Cfg::BN * 2;
  const char* out_wg = reinterpret_cast<const char*>(a.C) + (long)m0 * a.ldc * 2;
  uint32_t ooff[TM][4];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int it = 0; it < 4; ++it) ooff[tm][it] = (uint32_t)(wm * Cfg::WM + tm * 32 + 8 * it + er) * row_stride + (wn * Cfg::WN + ec * 8) * 2;

  const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  f32x16_t acc[TN][TM];
  auto epilogue = [&](int step) {
    const uint64_t out_step = reinterpret_cast<uint64_t>(out_wg + (long)step * step_stride);
    i32x4_t sent[TM][4];
    static_for<0, TM>([&](auto tmc) {
      constexpr int tm = decltype(tmc)::value;
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = acc[tn][tm][4 * rq + e] * descale;
            // (keeps the fp32 product a value of its own: fused with the conversion to f16 it is rounded once, not twice
            // as in the kernels whose product passes through an epilogue first, and 0.05 % of the outputs differ)
            if constexpr (OUT_DT == DT_F16) asm volatile("" : "+v"(v[e]));
          }
          u32x2_t w2;
          if constexpr (OUT_DT == DT_BF16) w2 = u32x2_t{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          else w2 = u32x2_t{(uint32_t)f32_to_f16_bits(v[0]) | ((uint32_t)f32_to_f16_bits(v[1]) << 16),
                            (uint32_t)f32_to_f16_bits(v[2]) | ((uint32_t)f32_to_f16_bits(v[3]) << 16)};
          const uint32_t waddr = pw[(tn << 2) | rq];   // (operands of an asm statement inside a generic lambda must be its own locals)
          asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(waddr), "v"(w2), "n"(tm * Cfg::PATCH_BYTES) : "memory");
        }
      // (LDS executes a wave's operations in order: the reads below see the writes above)
      // (one statement with its wait inside: an output of an asm statement counts as ready when the statement ends)
      i32x4_t q[4];
      const uint32_t raddr = pr;
      asm volatile(
          "ds_read_b128 %0, %4 offset:%5\n\tds_read_b128 %1, %4 offset:%6\n\tds_read_b128 %2, %4 offset:%7\n\tds_read_b128 %3, %4 offset:%8\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(q[0]), "=&v"(q[1]), "=&v"(q[2]), "=&v"(q[3])
          : "v"(raddr), "n"(tm * Cfg::PATCH_BYTES), "n"(tm * Cfg::PATCH_BYTES + 1024), "n"(tm * Cfg::PATCH_BYTES + 2048), "n"(tm * Cfg::PATCH_BYTES + 3072)
          : "memory");
      // The halves of odd row groups are exchanged into registers of their own before the first store, and all four
      // data vectors stay alive until the end of the epilogue: a 16-byte store reads its data registers some cycles after
      // it issues, the compiler keeps that distance only for stores it generates itself, and overwriting them in the
      // next instruction but one (a nop in between) still sent stale lanes to memory.
      const i32x4_t x1 = {q[1][2], q[1][3], q[1][0], q[1][1]}, x3 = {q[3][2], q[3][3], q[3][0], q[3][1]};
      const uint32_t o0 = ooff[tm][0], o1 = ooff[tm][1], o2 = ooff[tm][2], o3 = ooff[tm][3];
      const uint64_t base = out_step;
      asm volatile(
          "global_store_dwordx4 %0, %4, %8 nt\n\tglobal_store_dwordx4 %1, %5, %8 nt\n\t"
          "global_store_dwordx4 %2, %6, %8 nt\n\tglobal_store_dwordx4 %3, %7, %8 nt"
          ::"v"(o0), "v"(o1), "v"(o2), "v"(o3), "v"(q[0]), "v"(x1), "v"(q[2]), "v"(x3), "s"(base)
          : "memory");
      sent[tm][0] = q[0]; sent[tm][1] = x1; sent[tm][2] = q[2]; sent[tm][3] = x3;
    });
    // (the end of the data registers' lives: both strips' stores are behind, the first by a whole strip)
    asm volatile("s_nop 7" ::"v"(sent[0][0]), "v"(sent[0][1]), "v"(sent[0][2]), "v"(sent[0][3]),
                 "v"(sent[1][0]), "v"(sent[1][1]), "v"(sent[1][2]), "v"(sent[1][3]));
  };

  // The loop is rotated: iteration `step` writes out the result of step - 1 and then multiplies step. The wait in
  // front of the barrier has to be for everything (loads and stores retire in no fixed order with respect to each
  // other, so no count separates this step's weights from the stores before them); placed like this it finds the
  // stores a whole MFMA phase old and the weights an epilogue and an MFMA phase old.
  for (int step = 0; step <= nsteps; ++step) {
    wait_vmcnt<0>();
    dmam_barrier();
    // Every wave has read the other stage for the last time before it reached this barrier.
    issue_step(step + 1);
    if (step > 0) epilogue(step - 1);
    if (step == nsteps) break;
    const uint32_t stage_off = (step & 1) * Cfg::STAGE_BYTES;
    static_for<0, KSTEPS>([&](auto ksc) {
      constexpr int ks = decltype(ksc)::value;
      Frag<DT_FP8> wf[TN];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        wf[tn].lo = read_w(stage_off, tn, ks, 0);
        wf[tn].hi = read_w(stage_off, tn, ks, 1);
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = mfma_frag<DT_FP8>(wf[tn], xf[tm][ks], ks == 0 ? zero : acc[tn][tm]);
    });
  }
  wait_vmcnt<0>();   // (the empty loads past the last step)
}

template <int OUT_DT>
static hipError_t launch_shortk(const GemmArgs& a, hipStream_t st) {
  static std::atomic<bool> attr_set[16] = {};
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_shortk_kernel<OUT_DT>;
  if (!attr_set[dev]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, ShortKCfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  hipLaunchKernelGGL(kern, dim3((a.M + ShortKCfg::BM - 1) / ShortKCfg::BM), dim3(ShortKCfg::NT), ShortKCfg::LDS_BYTES, st, a);
  return hipGetLastError();
}

}  // namespace crl
