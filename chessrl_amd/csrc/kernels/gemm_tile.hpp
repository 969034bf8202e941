// Device code shared by the GEMM kernels of gemm.hip (register-staged 64x64 / 128x128 tiles) and gemm_dma.hip
// (256x256 tile fed by direct global->LDS loads): MFMA operand fragments read from swizzled LDS rows, the output
// stores, and the epilogue C = res + alpha*act(descale*acc + bias) with its amax, fp8 scaling and C/C2 split.
#pragma once
#include <type_traits>

#include "common.hpp"

namespace crl {

__device__ __forceinline__ int lds_swizzle(int row) { return (row ^ (row >> 3)) & 7; }

// Compile-time loop: f is called with std::integral_constant<int, I> for I in [0, N), so
// register arrays indexed by I never need dynamic indexing whatever the body size.
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// One MFMA operand fragment of a lane: 16 bytes (2-byte types, 8 k-elements) or
// 32 bytes (fp8, 32 k-elements) of one LDS row.
template <int IN_DT>
struct Frag {
  i32x4_t lo;
};
template <>
struct Frag<DT_FP8> {
  i32x4_t lo, hi;
};

template <int IN_DT>
__device__ __forceinline__ Frag<IN_DT> load_frag(const uint8_t* row, int sw, int ks, int g) {
  Frag<IN_DT> f;
  if constexpr (IN_DT == DT_FP8) {
    const int c0 = 4 * ks + 2 * g;
    f.lo = *reinterpret_cast<const i32x4_t*>(row + ((c0 ^ sw) << 4));
    f.hi = *reinterpret_cast<const i32x4_t*>(row + (((c0 + 1) ^ sw) << 4));
  } else {
    const int c0 = 2 * ks + g;
    f.lo = *reinterpret_cast<const i32x4_t*>(row + ((c0 ^ sw) << 4));
  }
  return f;
}

template <int IN_DT>
__device__ __forceinline__ f32x16_t mfma_frag(const Frag<IN_DT>& w, const Frag<IN_DT>& x, f32x16_t acc) {
  if constexpr (IN_DT == DT_FP8) {
    i32x8_t wv = {w.lo[0], w.lo[1], w.lo[2], w.lo[3], w.hi[0], w.hi[1], w.hi[2], w.hi[3]};
    i32x8_t xv = {x.lo[0], x.lo[1], x.lo[2], x.lo[3], x.hi[0], x.hi[1], x.hi[2], x.hi[3]};
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wv, xv, acc, 0, 0, 0, 0, 0, 0);
  } else if constexpr (IN_DT == DT_BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, w.lo), __builtin_bit_cast(bf16x8_t, x.lo), acc, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, w.lo), __builtin_bit_cast(f16x8_t, x.lo), acc, 0, 0, 0);
  }
}

template <int OUT_DT>
__device__ __forceinline__ void store1(void* base, long off, float v) {
  if constexpr (OUT_DT == DT_F32) reinterpret_cast<float*>(base)[off] = v;
  else if constexpr (OUT_DT == DT_BF16) reinterpret_cast<uint16_t*>(base)[off] = f32_to_bf16_bits(v);
  else if constexpr (OUT_DT == DT_F16) reinterpret_cast<uint16_t*>(base)[off] = f32_to_f16_bits(v);
  else reinterpret_cast<uint8_t*>(base)[off] = f32_to_fp8(v);
}

// Orders this wave's LDS traffic (LDS executes one wave's operations in issue order) and
// keeps the compiler from moving accesses across the point.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// 16 bytes read once (a 16-bit residual row segment): loaded with the non-temporal hint so that it does not displace
// the operand tiles the workgroups of an XCD share in L2 (an fp32 residual stream measured 2 % slower with the hint
// and keeps plain loads).
__device__ __forceinline__ uint4 nt_load16(const char* p) {
  const i32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const i32x4_t*>(p));
  return make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
}

// NT: store with the non-temporal hint, so a streamed output does not evict the operands from L2.
template <int OUT_DT, int NT = 0>
__device__ __forceinline__ void store8(void* base, long off, const float v[8]) {
  // The hint is written as an instruction: __builtin_nontemporal_store beside a plain store of the same value in the
  // other arm of a branch is merged with it by the compiler, and the hint is dropped. The idle cycles behind it keep the
  // next writer of the data registers away: a 16-byte store reads them some cycles after it issues, and the compiler,
  // which knows that of its own stores, cannot see this one.
  auto put = [](i32x4_t* p, i32x4_t x) {
    if constexpr (NT) asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 7" ::"v"(p), "v"(x) : "memory");
    else *p = x;
  };
  if constexpr (OUT_DT == DT_F32) {
    i32x4_t* p = reinterpret_cast<i32x4_t*>(reinterpret_cast<float*>(base) + off);
    put(p, i32x4_t{(int)__float_as_uint(v[0]), (int)__float_as_uint(v[1]), (int)__float_as_uint(v[2]), (int)__float_as_uint(v[3])});
    put(p + 1, i32x4_t{(int)__float_as_uint(v[4]), (int)__float_as_uint(v[5]), (int)__float_as_uint(v[6]), (int)__float_as_uint(v[7])});
  } else if constexpr (OUT_DT == DT_BF16) {
    put(reinterpret_cast<i32x4_t*>(reinterpret_cast<uint16_t*>(base) + off),
        i32x4_t{(int)pack_bf16x2(v[0], v[1]), (int)pack_bf16x2(v[2], v[3]), (int)pack_bf16x2(v[4], v[5]), (int)pack_bf16x2(v[6], v[7])});
  } else if constexpr (OUT_DT == DT_F16) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_f16_bits(v[2 * i]) | ((uint32_t)f32_to_f16_bits(v[2 * i + 1]) << 16);
    put(reinterpret_cast<i32x4_t*>(reinterpret_cast<uint16_t*>(base) + off), i32x4_t{(int)w[0], (int)w[1], (int)w[2], (int)w[3]});
  } else {
    typedef int i32x2_t __attribute__((ext_vector_type(2)));
    const i32x2_t x = {(int)pack_fp8x4(v[0], v[1], v[2], v[3]), (int)pack_fp8x4(v[4], v[5], v[6], v[7])};
    i32x2_t* p = reinterpret_cast<i32x2_t*>(reinterpret_cast<uint8_t*>(base) + off);
    if constexpr (NT) asm volatile("global_store_dwordx2 %0, %1, off nt" ::"v"(p), "v"(x) : "memory");
    else *p = x;
  }
}

// 8 values as 16 bytes of a 16-bit type (all four dwords) or 8 bytes of e4m3 (the first two dwords).
template <int OUT_DT>
__device__ __forceinline__ i32x4_t pack8(const float v[8]) {
  static_assert(OUT_DT != DT_F32, "converted outputs only");
  if constexpr (OUT_DT == DT_BF16) {
    return i32x4_t{(int)pack_bf16x2(v[0], v[1]), (int)pack_bf16x2(v[2], v[3]), (int)pack_bf16x2(v[4], v[5]), (int)pack_bf16x2(v[6], v[7])};
  } else if constexpr (OUT_DT == DT_F16) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_f16_bits(v[2 * i]) | ((uint32_t)f32_to_f16_bits(v[2 * i + 1]) << 16);
    return i32x4_t{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
  } else {
    return i32x4_t{(int)pack_fp8x4(v[0], v[1], v[2], v[3]), (int)pack_fp8x4(v[4], v[5], v[6], v[7]), 0, 0};
  }
}

// Shared epilogue. acc[tn][tm][r] is output row m = mw0 + tm*32 + lr, column
// n = nw0 + tn*32 + 8*(r/4) + 4*g + (r%4) (lr = lane%32, g = lane/32); sC is this wave's
// private LDS patch of 32 x WN floats.
//
// Each 32 x WN strip of the wave tile goes through the patch (16-byte chunks XOR-swizzled by
// row) so that a lane ends up with 8 consecutive columns of one row: stores, residual loads
// and bias loads are 16-byte vectors (32 for fp32) and every store instruction writes whole
// row segments. A lane keeps the same 8 columns for all rows, so its bias is loaded once. The
// residual of strip t+1 is requested before strip t is processed (two register sets), which
// takes its memory latency off the critical path; the activation is selected once per strip.
//
// The branches for tiles that hang over an edge of C or meet an unaligned row stride are marked unlikely, so that the
// compiler moves them out of the straight path. Left inline between the vector accesses they put a taken jump over a
// kilobyte of cold code in front of every store and residual load; identical kernels then ran 5-10 % apart depending
// on where the code object happened to place them (instruction-cache misses at the jump targets), and 5 % slower than
// this form at best. (A second, compile-time variant of the epilogue for tiles entirely inside C was tried on top:
// two inlined copies push the 256x256 kernel into register spills.)
// RES_NORM: the 16-bit residual is normalised on the fly, LayerNorm(res) = (res * s0_m + s1_m) * gain_n + offset_n with
// s0 = 1/std and s1 = -mean/std of row m, from the row statistics a.res_stats and the norm's gain and offset (the normalised tensor then never travels
// through memory). sStats: 2*WM floats of LDS of this wave's own for its rows' statistics, filled here (RES_NORM 1)
// or by the kernel before its main loop (RES_NORM 2).
// LEAN (the launcher says when): every row of the tile is inside C, N and nsplit are multiples of 8 with 16-byte aligned
// rows everywhere, a residual (if any) is bf16 with one row per output row, and no maximum is asked for; the row and
// alignment guards, the scalar edge stores, the fp32/f16 residual blocks and the maximum then are not in the code at all.
// LEAN == 2 on top of that fixes what the call does at compile time: no activation (for an e4m3 output: the fused mish and
// nothing else), a residual exactly when RES_NORM says so, alpha = 1 without one, a streamed output.
template <int WM, int WN, int OUT_DT, int RES_NORM = 0, int LEAN = 0, typename AccArr>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& a, AccArr& acc, float* sC, int mw0, int nw0, int lane,
                                              float* sStats = nullptr, const float* sCols = nullptr) {
  // sCols (optional, LDS): per-column constants of this wave's WN columns that the kernel has staged before its main
  // loop, so that the epilogue does not start by waiting for global memory: bias at [0, WN), and for RES_NORM the
  // residual gain at [WN, 2 WN) and offset at [2 WN, 3 WN) (the parts whose pointers are null are not read).
  // acc is f32x16_t[WN/32][WM/32] (32x32 MFMA tiles) or f32x4_t[WN/16][WM/16] (16x16 tiles).
  constexpr bool MI16 = sizeof(acc[0][0]) == sizeof(f32x4_t);
  constexpr bool EXACT = LEAN == 2;
  constexpr int TM = WM / 32, TN = WN / 32, CH4 = WN / 4, CP = WN / 8, RSTEP = 64 / CP, ITERS = 32 / RSTEP;
  const int lr = lane & 31, g = lane >> 5;
  const int ec = lane % CP, er = lane / CP;
  const int n = nw0 + ec * 8;
  const bool n_ok = n < a.N;
  const bool full = LEAN ? true : a.vec_ok && (n + 7 < a.N) && ((n < a.nsplit) == (n + 7 < a.nsplit));
  float bias8[8];
  if (sCols != nullptr) {
    if (a.bias) {
      const f32x4_t b0 = *reinterpret_cast<const f32x4_t*>(sCols + ec * 8), b1 = *reinterpret_cast<const f32x4_t*>(sCols + ec * 8 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { bias8[e] = b0[e]; bias8[4 + e] = b1[e]; }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) bias8[e] = 0.f;
    }
  } else if (__builtin_expect(a.bias != nullptr && n + 7 < a.N && (reinterpret_cast<uintptr_t>(a.bias) & 15) == 0, 1)) {
    const f32x4_t b0 = *reinterpret_cast<const f32x4_t*>(a.bias + n), b1 = *reinterpret_cast<const f32x4_t*>(a.bias + n + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { bias8[e] = b0[e]; bias8[4 + e] = b1[e]; }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) bias8[e] = (a.bias && n + e < a.N) ? a.bias[n + e] : 0.f;
  }
  const int res_dt = LEAN ? (int)DT_BF16 : a.res_dtype;
  const float descale = a.descale, alpha = a.alpha;
  float local_amax = 0.f;
  // e4m3(out_scale * mish(descale * acc + bias)) with nothing else asked for (the FFN's first product): the activation in
  // 15.5 instead of 19.5 instruction slots per element (a transcendental counts four), which matters because both waves of
  // a SIMD sit in this code at once with the matrix pipe idle (0.45 us per slot and 256x256 tile). With n = e^x,
  // mish(x) = x (1 - 2 / (n (n + 2) + 2)): x log2(e) comes straight from the accumulator by a fused multiply-add of its
  // own, out_scale rides on the factor, and no clamp of the exponent is needed (n = inf gives the factor 1).
  // The difference 1 - 2r loses relative accuracy only where mish itself is below 1e-3 of its argument; the 16-bit outputs keep act_mish.
  bool fused_mish = false;
  float bias_l2[8], d_l2 = 0.f, os_m2 = 0.f, os_1 = 0.f;
  if constexpr (OUT_DT == DT_FP8) {
    fused_mish = EXACT || (a.act == ACT_MISH && !a.res && alpha == 1.f && !a.amax);
    if (fused_mish) {
      constexpr float L2E = 1.4426950408889634f;
      os_1 = a.out_scale; os_m2 = -2.f * os_1;
      d_l2 = descale * L2E;
#pragma unroll
      for (int e = 0; e < 8; ++e) bias_l2[e] = bias8[e] * L2E;
    }
  }
  float gain8[8];
  if constexpr (RES_NORM) {
    // offset_n joins the bias (which is multiplied by alpha below); the statistics of this wave's rows go to LDS.
    const float inv_alpha = 1.0f / alpha;
    if (sCols != nullptr) {
      const f32x4_t g0 = *reinterpret_cast<const f32x4_t*>(sCols + WN + ec * 8), g1 = *reinterpret_cast<const f32x4_t*>(sCols + WN + ec * 8 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { gain8[e] = g0[e]; gain8[4 + e] = g1[e]; }
      if (a.res_beta) {
        const f32x4_t o0 = *reinterpret_cast<const f32x4_t*>(sCols + 2 * WN + ec * 8), o1 = *reinterpret_cast<const f32x4_t*>(sCols + 2 * WN + ec * 8 + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { bias8[e] += o0[e] * inv_alpha; bias8[4 + e] += o1[e] * inv_alpha; }
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const bool ok = n + e < a.N;
        gain8[e] = ok ? a.res_gamma[n + e] : 0.f;
        if (a.res_beta && ok) bias8[e] += a.res_beta[n + e] * inv_alpha;
      }
    }
    if constexpr (RES_NORM == 1) {   // (2: the kernel has staged them before its main loop)
#pragma unroll
      for (int r = lane; r < WM; r += 64) {
        const int m = mw0 + r;
        const float2 st = m < a.M ? *reinterpret_cast<const float2*>(a.res_stats + 2 * (long)m) : make_float2(0.f, 0.f);
        *reinterpret_cast<float2*>(sStats + 2 * r) = st;
      }
      wave_lds_fence();
    }
  }
  // A lane keeps its 8 columns for every row, so which output (C or C2), the column inside it and the row stride are
  // fixed per lane: the vector paths address row m as base + m * stride.
  constexpr int OUT_SZ = OUT_DT == DT_F32 ? 4 : OUT_DT == DT_FP8 ? 1 : 2;
  const bool first = n < a.nsplit;
  char* const out_base = reinterpret_cast<char*>(first ? a.C : a.C2) + (long)(first ? n : n - a.nsplit) * OUT_SZ;
  const long out_stride = (first ? a.ldc : a.ldc2) * OUT_SZ;
  const int res_sz = res_dt == DT_F32 ? 4 : 2;
  const char* const res_base = reinterpret_cast<const char*>(a.res) + (long)n * res_sz;
  const long res_stride = a.ldr * res_sz;

  // Raw residual bits, 16 bytes per step and set. 16-bit residuals use the two sets as a double
  // buffer over strips; an fp32 residual (8 values = 32 bytes) uses both sets for the current
  // strip (low and high half), i.e. it is fetched at the start of its own strip.
  const bool res32 = LEAN ? false : res_dt == DT_F32;
  uint4 rraw[2][ITERS];
  // LEAN: rows are visited in order, RSTEP apart, by the residual loads and by the stores alike, so each keeps a running
  // pointer (one 64-bit add per access where base + row * stride costs a 64-bit multiply-add and its two 32-bit products).
  const char* res_cur = res_base + (long)(mw0 + er) * res_stride;
  const long res_step = RSTEP * res_stride;
  char* out_cur = out_base + (long)(mw0 + er) * out_stride;
  const long out_step = RSTEP * out_stride;
  auto load_res = [&](int tm, int set, int half) {
    if constexpr (LEAN) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        rraw[set][it] = n_ok ? nt_load16(res_cur) : make_uint4(0, 0, 0, 0);
        res_cur += res_step;
      }
      return;
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int m = mw0 + tm * 32 + er + it * RSTEP;
      uint4 val = make_uint4(0, 0, 0, 0);
      if (__builtin_expect((LEAN || m < a.M) && n_ok, 1)) {
        const long rrow = (!LEAN && a.res_rows > 0) ? m % a.res_rows : m;
        const long ro = rrow * a.ldr + n;
        if (res32) {
          const float* rp = reinterpret_cast<const float*>(a.res) + ro + 4 * half;
          if (__builtin_expect(full, 1)) val = *reinterpret_cast<const uint4*>(res_base + rrow * res_stride + 16 * half);
          else {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (n + 4 * half + e < a.N) ? __float_as_uint(rp[e]) : 0u;
            val = make_uint4(w[0], w[1], w[2], w[3]);
          }
        } else {
          const uint16_t* rp = reinterpret_cast<const uint16_t*>(a.res) + ro;
          if (__builtin_expect(full, 1)) val = nt_load16(res_base + rrow * res_stride);
          else {
            uint32_t h[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) h[e] = (n + e < a.N) ? (uint32_t)rp[e] : 0u;
            val = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
          }
        }
      }
      rraw[set][it] = val;
    }
  };
  const bool has_res = EXACT ? RES_NORM != 0 : a.res != nullptr;
  if (has_res && !res32) load_res(0, 0, 0);
  static_for<0, TM>([&](auto tmc) {
    constexpr int tm = decltype(tmc)::value;
    if (has_res) {
      if (res32) { load_res(tm, 0, 0); load_res(tm, 1, 1); }
      else if constexpr (tm + 1 < TM) load_res(tm + 1, (tm + 1) & 1, 0);
    }
    if constexpr (MI16) {
      // A 16x16 tile holds, per lane, columns 4 (lane / 16) + {0..3} of row lane % 16: one 16-byte chunk of the patch row.
#pragma unroll
      for (int wi = 0; wi < WN / 16; ++wi)
#pragma unroll
        for (int xi = 0; xi < 2; ++xi) {
          const int row = 16 * xi + (lane & 15), chunk = wi * 4 + (lane >> 4);
          *reinterpret_cast<f32x4_t*>(sC + row * WN + ((chunk ^ (row & (CH4 - 1))) << 2)) = acc[wi][2 * tm + xi];
        }
    } else {
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int chunk = tn * 8 + 2 * rq + g;
          f32x4_t v4 = {acc[tn][tm][4 * rq], acc[tn][tm][4 * rq + 1], acc[tn][tm][4 * rq + 2], acc[tn][tm][4 * rq + 3]};
          *reinterpret_cast<f32x4_t*>(sC + lr * WN + ((chunk ^ (lr & (CH4 - 1))) << 2)) = v4;
        }
    }
    wave_lds_fence();
    float v[ITERS][8];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int r = er + it * RSTEP;
      const int sw = r & (CH4 - 1);
      const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(sC + r * WN + (((2 * ec) ^ sw) << 2));
      const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(sC + r * WN + (((2 * ec + 1) ^ sw) << 2));
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[it][e] = fmaf(lo[e], descale, bias8[e]);
        v[it][4 + e] = fmaf(hi[e], descale, bias8[4 + e]);
      }
      if constexpr (OUT_DT == DT_FP8) {
        if (fused_mish) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float accv = e < 4 ? lo[e] : hi[e - 4];
            const float nexp = __builtin_amdgcn_exp2f(fmaf(accv, d_l2, bias_l2[e]));
            const float w = fmaf(nexp, nexp + 2.f, 2.f);
            v[it][e] *= fmaf(fast_rcp(w), os_m2, os_1);
          }
        }
      }
    }
    if (fused_mish) goto store_strip;
    if constexpr (!EXACT) switch (a.act) {  // uniform
      case ACT_GELU:
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
          for (int e = 0; e < 8; ++e) v[it][e] = act_gelu(v[it][e]);
        break;
      case ACT_MISH:
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
          for (int e = 0; e < 8; ++e) v[it][e] = act_mish(v[it][e]);
        break;
      case ACT_SWISH:
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
          for (int e = 0; e < 8; ++e) v[it][e] = act_swish(v[it][e]);
        break;
      default: break;
    }
    if (has_res) {
      // One straight block per residual type (the type test per element compiles to a chain of branches).
      if (res32) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const uint4 lo = rraw[0][it], hi = rraw[1][it];
          const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
          for (int e = 0; e < 8; ++e) v[it][e] = fmaf(v[it][e], alpha, __uint_as_float(w[e]));
        }
      } else if (res_dt == DT_F16) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const uint4 q = rraw[tm & 1][it];
          const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[it][e] = fmaf(v[it][e], alpha, f16_bits_to_f32((uint16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffff))));
        }
      } else if constexpr (RES_NORM) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const uint4 q = rraw[tm & 1][it];
          const uint32_t w[4] = {q.x, q.y, q.z, q.w};
          const float2 st = *reinterpret_cast<const float2*>(sStats + 2 * (tm * 32 + er + it * RSTEP));
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float r = __uint_as_float((e & 1) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16));
            v[it][e] = fmaf(v[it][e], alpha, fmaf(r, st.x, st.y) * gain8[e]);
          }
        }
      } else {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const uint4 q = rraw[tm & 1][it];
          const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[it][e] = fmaf(v[it][e], alpha, __uint_as_float((e & 1) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16)));
        }
      }
    } else if (!EXACT && alpha != 1.f) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[it][e] *= alpha;
    }
    if (!LEAN && a.amax) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (mw0 + tm * 32 + er + it * RSTEP < a.M && n + e < a.N) local_amax = fmaxf(local_amax, fabsf(v[it][e]));
    }
    if constexpr (OUT_DT == DT_FP8) {
      const float os = a.out_scale;
#pragma unroll
      for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[it][e] *= os;
    }
  store_strip:

    if constexpr (LEAN != 0 && OUT_DT != DT_F32) {
      // All of the strip's vectors are converted into registers of their own before the first store and kept alive past
      // the last: a 16-byte store written as inline assembly reads its data some cycles after it issues, the compiler
      // keeps that distance only for stores it generates itself, and in code this tight the next conversion would land in
      // the registers of a store still reading them.
      i32x4_t x[ITERS];
#pragma unroll
      for (int it = 0; it < ITERS; ++it) x[it] = pack8<OUT_DT>(v[it]);
      if (n_ok) {
        if (EXACT || a.stream_out) {
#pragma unroll
          for (int it = 0; it < ITERS; ++it) {
            if constexpr (OUT_DT == DT_FP8) {
              typedef int i32x2_t __attribute__((ext_vector_type(2)));
              const i32x2_t x2 = {x[it][0], x[it][1]};
              asm volatile("global_store_dwordx2 %0, %1, off nt" ::"v"(out_cur), "v"(x2) : "memory");
            } else {
              asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(out_cur), "v"(x[it]) : "memory");
            }
            out_cur += out_step;
          }
        } else {
#pragma unroll
          for (int it = 0; it < ITERS; ++it) {
            if constexpr (OUT_DT == DT_FP8) {
              typedef int i32x2_t __attribute__((ext_vector_type(2)));
              *reinterpret_cast<i32x2_t*>(out_cur) = i32x2_t{x[it][0], x[it][1]};
            } else {
              *reinterpret_cast<i32x4_t*>(out_cur) = x[it];
            }
            out_cur += out_step;
          }
        }
      } else {
        out_cur += ITERS * out_step;
      }
      static_assert(ITERS == 4 || ITERS == 2 || ITERS == 8, "strip shapes of the tiled kernels");
      if constexpr (ITERS == 4) asm volatile("s_nop 7" ::"v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]));
      else if constexpr (ITERS == 2) asm volatile("s_nop 7" ::"v"(x[0]), "v"(x[1]));
      else asm volatile("s_nop 7" ::"v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(x[4]), "v"(x[5]), "v"(x[6]), "v"(x[7]));
    } else
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int m = mw0 + tm * 32 + er + it * RSTEP;
      if constexpr (LEAN != 0) {
        if (n_ok) {
          if (EXACT || a.stream_out) store8<OUT_DT, 1>(out_cur, 0, v[it]);
          else store8<OUT_DT, 0>(out_cur, 0, v[it]);
        }
        out_cur += out_step;
        continue;
      }
      if (__builtin_expect((!LEAN && m >= a.M) || !n_ok, 0)) continue;
      if (__builtin_expect(full, 1)) {
        char* dst = out_base + m * out_stride;
        if (a.stream_out) store8<OUT_DT, 1>(dst, 0, v[it]);
        else store8<OUT_DT, 0>(dst, 0, v[it]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if (n + e >= a.N) continue;
          if (n + e < a.nsplit) store1<OUT_DT>(a.C, (long)m * a.ldc + n + e, v[it][e]);
          else store1<OUT_DT>(a.C2, (long)m * a.ldc2 + (n + e - a.nsplit), v[it][e]);
        }
      }
    }
    wave_lds_fence();
  });
  if (!LEAN && a.amax) {
    local_amax = wave_max(local_amax);
    if (lane == 0) atomic_amax(a.amax, local_amax);
  }
}

// The 256x256 direct-to-LDS tile (gemm_dma.hip). It lives in a translation unit, and so a device code object, of its
// own: its speed depends measurably on where its code lands (identical instructions ran 3-8 % slower after unrelated
// kernels were added to the same code object), and alone it stays where it was measured.
hipError_t launch_gemm_dma(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st);
// One 256-byte block of zeros per device (gemm.hip): the source of K-tail chunks for the direct-to-LDS loads.
const uint8_t* device_zeros(hipError_t* err);
hipError_t launch_gemm_dma_resnorm(const GemmArgs& a, hipStream_t st);   // gemm_dma_resnorm.hip
// gemm_dmaf.hip: the eight-wave in-step tile with address arithmetic kept out of the main loop (K in whole 128-byte slabs).
bool gemm_dmaf_has(int in_dt, int out_dt, bool res_norm);
hipError_t launch_gemm_dmaf(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st);
// gemm_dmam.hip: the 128x128 tile fed by direct-to-LDS loads through a four-stage ring (K in whole 128-byte slabs, no normalised residual).
bool gemm_dmam_has(int in_dt, int out_dt);
hipError_t launch_gemm_dmam(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st, int tile_size);
// gemm_shortk.hip: K = 256 e4m3 operands, bare scaled product: a workgroup keeps 256 rows of A in registers and walks N.
bool gemm_shortk_can(const GemmArgs& a, int in_dt, int out_dt);
hipError_t launch_gemm_shortk(const GemmArgs& a, int in_dt, int out_dt, hipStream_t st);
// gemm_sp2.hip: the same four waves fed in 128-byte slabs of K.
hipError_t launch_gemm_sp2(const GemmArgs& a, int out_dt, hipStream_t st);

}  // namespace crl
