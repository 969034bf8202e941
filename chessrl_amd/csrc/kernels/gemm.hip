// C[M,N] = epilogue(A[M,K] · W[N,K]^T) on the gfx950 matrix cores.
//
// Replaces the nn.Linear call sites of the reference forward
// (model_bis.py:42,44,89,91,139; new_paradigm/attn.py:478-489; new_paradigm/value.py:39-40,
// 129-152,423-425) and the fp8 te.Linear sites of model_fp8.py:43,45,90,92,140.
//
// Layout of the work:
//  * Both operands are K-contiguous, so a K-slab of 128 bytes per row (64 bf16/f16 or
//    128 fp8 elements) is staged in LDS for BM activation rows and BN weight rows. The
//    kernel is written on bytes: one code path serves 2-byte and 1-byte element types.
//  * LDS rows are 128 bytes = 8 chunks of 16 bytes; chunk c of row r is stored at
//    chunk c ^ ((r ^ (r>>3)) & 7), which keeps both the 16-byte fragment reads and the
//    row-wise stores free of bank conflicts (measured: SQ_LDS_BANK_CONFLICT = 0).
//  * Each wave owns a (WM x WN) sub-tile made of 32x32 MFMA tiles. The weight rows are
//    the MFMA row operand and the activation rows the column operand, so a lane ends
//    up holding four consecutive output columns of one output row, which the epilogue
//    moves through LDS as 16-byte chunks.
//  * Global loads for slab k+1 are issued before the MFMAs of slab k and written to LDS
//    afterwards (register staging). With two LDS stages that costs one barrier per slab;
//    the single-stage variant uses two barriers and half the LDS so two workgroups fit
//    on a CU and cover each other's stalls.
//  * Workgroup ids are remapped so each XCD (ids round-robin over 8 XCDs) walks a
//    contiguous range of tiles, N fastest: the weight matrix stays in that XCD's L2
//    and every activation slab is fetched from HBM by one XCD only.
#include <type_traits>

#include "common.hpp"

namespace crl {

template <int BM_, int BN_, int WGM_, int WGN_, int STAGES_, int FRAG_DB_, int MIN_WAVES_>
struct GemmCfg {
  static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_, STAGES = STAGES_, FRAG_DB = FRAG_DB_;
  static constexpr int MIN_WAVES = MIN_WAVES_;
  static constexpr int NW = WGM * WGN, NT = 64 * NW;
  static constexpr int WM = BM / WGM, WN = BN / WGN;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int ROWS_PER_PASS = NT / 8;
  static constexpr int A_PASSES = BM / ROWS_PER_PASS, W_PASSES = BN / ROWS_PER_PASS;
  static constexpr int STAGE_BYTES = (BM + BN) * 128;
  static constexpr int EPI_BYTES = NW * 32 * WN * 4;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES > EPI_BYTES ? STAGES * STAGE_BYTES : EPI_BYTES;
  static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile/threads mismatch");
  static_assert(WN >= 32 && WM >= 32, "wave tile too small");
};

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
__device__ __forceinline__ void store4(void* base, long off, const float v[4]) {
  if constexpr (OUT_DT == DT_F32) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(base) + off) = make_float4(v[0], v[1], v[2], v[3]);
  } else if constexpr (OUT_DT == DT_BF16) {
    uint2 p = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(base) + off) = p;
  } else if constexpr (OUT_DT == DT_F16) {
    uint2 p = make_uint2((uint32_t)f32_to_f16_bits(v[0]) | ((uint32_t)f32_to_f16_bits(v[1]) << 16),
                         (uint32_t)f32_to_f16_bits(v[2]) | ((uint32_t)f32_to_f16_bits(v[3]) << 16));
    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(base) + off) = p;
  } else {
    *reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(base) + off) = pack_fp8x4(v[0], v[1], v[2], v[3]);
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

template <typename Cfg, int IN_DT, int OUT_DT>
__global__ void __launch_bounds__(Cfg::NT, Cfg::MIN_WAVES) gemm_kernel(const GemmArgs a) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN;
  constexpr int ESZ = (IN_DT == DT_FP8) ? 1 : 2;
  constexpr int KSTEPS = (IN_DT == DT_FP8) ? 2 : 4;
  extern __shared__ __align__(16) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % Cfg::WGM, wn = wave / Cfg::WGM;
  const int lr = lane & 31, g = lane >> 5;

  // XCD-aware tile order.
  const int tiles_n = (a.N + BN - 1) / BN;
  const int nblk = gridDim.x;
  int pid = blockIdx.x;
  {
    const int per = nblk >> 3;  // full groups of 8
    if (pid < (per << 3)) pid = (pid & 7) * per + (pid >> 3);
  }
  const int tile_m = pid / tiles_n, tile_n = pid - tile_m * tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const long kbytes = (long)a.K * ESZ;
  const int nslab = (int)((kbytes + 127) >> 7);
  const uint8_t* Ab = reinterpret_cast<const uint8_t*>(a.A);
  const uint8_t* Wb = reinterpret_cast<const uint8_t*>(a.W);
  const long lda_b = a.lda * ESZ, ldw_b = a.ldw * ESZ;

  const int lchunk = tid & 7, lrow = tid >> 3;
  i32x4_t ra[Cfg::A_PASSES], rw[Cfg::W_PASSES];

  // Rows past M or N are clamped to the last valid row: they only feed output rows or
  // columns that are never stored, so no zero fill (and no branch) is needed.
  const uint8_t* aptr[Cfg::A_PASSES];
  const uint8_t* wptr[Cfg::W_PASSES];
#pragma unroll
  for (int i = 0; i < Cfg::A_PASSES; ++i) {
    int gm = m0 + lrow + i * Cfg::ROWS_PER_PASS;
    gm = gm < a.M ? gm : a.M - 1;
    aptr[i] = Ab + (long)gm * lda_b + (lchunk << 4);
  }
#pragma unroll
  for (int i = 0; i < Cfg::W_PASSES; ++i) {
    int gn = n0 + lrow + i * Cfg::ROWS_PER_PASS;
    gn = gn < a.N ? gn : a.N - 1;
    wptr[i] = Wb + (long)gn * ldw_b + (lchunk << 4);
  }
  // A K tail shorter than the slab is loaded from a clamped (valid) address and replaced by
  // zeros when the registers are written to LDS, i.e. after the wait that is needed there
  // anyway: nothing depends on the loaded data while the MFMAs of the current slab run.
  const long kmax = kbytes - 16;  // last valid 16-byte chunk offset along K
  const long kmine = lchunk << 4;
  auto gload = [&](int slab) {
    const long kb = ((long)slab << 7);
    const long kofs = (kb + kmine <= kmax) ? kb : kmax - kmine;
#pragma unroll
    for (int i = 0; i < Cfg::A_PASSES; ++i) ra[i] = *reinterpret_cast<const i32x4_t*>(aptr[i] + kofs);
#pragma unroll
    for (int i = 0; i < Cfg::W_PASSES; ++i) rw[i] = *reinterpret_cast<const i32x4_t*>(wptr[i] + kofs);
  };
  auto sstore = [&](int stage, int slab) {
    uint8_t* sW = smem + stage * Cfg::STAGE_BYTES;
    uint8_t* sA = sW + BN * 128;
    const bool kok = ((long)slab << 7) + kmine <= kmax;
    const i32x4_t z = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < Cfg::A_PASSES; ++i) {
      const int r = lrow + i * Cfg::ROWS_PER_PASS;
      *reinterpret_cast<i32x4_t*>(sA + r * 128 + ((lchunk ^ lds_swizzle(r)) << 4)) = kok ? ra[i] : z;
    }
#pragma unroll
    for (int i = 0; i < Cfg::W_PASSES; ++i) {
      const int r = lrow + i * Cfg::ROWS_PER_PASS;
      *reinterpret_cast<i32x4_t*>(sW + r * 128 + ((lchunk ^ lds_swizzle(r)) << 4)) = kok ? rw[i] : z;
    }
  };

  f32x16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // LDS rows this lane reads its fragments from (fixed for the whole kernel).
  int wrow_off[TN], wrow_sw[TN], arow_off[TM], arow_sw[TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int wr = wn * Cfg::WN + tn * 32 + lr;
    wrow_off[tn] = wr * 128;
    wrow_sw[tn] = lds_swizzle(wr);
  }
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int ar = wm * Cfg::WM + tm * 32 + lr;
    arow_off[tm] = BN * 128 + ar * 128;
    arow_sw[tm] = lds_swizzle(ar);
  }

  gload(0);
  sstore(0, 0);
  __syncthreads();

  // With FRAG_DB two fragment sets alternate: while the MFMAs of k-step ks run on one set,
  // the LDS reads of k-step ks+1 fill the other; the scheduling barriers keep that order
  // (left alone the compiler reuses one register set and exposes the LDS latency before
  // every MFMA group). Without it one set is used and a second resident wave hides the latency.
  // (fp8 fragments are twice as large: two sets would not fit beside 256 accumulators.)
  constexpr bool FRAG_DB = Cfg::FRAG_DB && IN_DT != DT_FP8;
  constexpr int NSET = FRAG_DB ? 2 : 1;
  Frag<IN_DT> wf[NSET][TN], xf[NSET][TM];
  auto lds_frags = [&](const uint8_t* st, int ks, int set) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) wf[set][tn] = load_frag<IN_DT>(st + wrow_off[tn], wrow_sw[tn], ks, g);
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) xf[set][tm] = load_frag<IN_DT>(st + arow_off[tm], arow_sw[tm], ks, g);
  };
  auto mfmas = [&](int set) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = mfma_frag<IN_DT>(wf[set][tn], xf[set][tm], acc[tn][tm]);
  };

  for (int slab = 0; slab < nslab; ++slab) {
    const int stage = Cfg::STAGES == 2 ? (slab & 1) : 0;
    const uint8_t* st = smem + stage * Cfg::STAGE_BYTES;
    const bool more = slab + 1 < nslab;
    if (more) gload(slab + 1);
    if constexpr (FRAG_DB) {
      lds_frags(st, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        if (ks + 1 < KSTEPS) lds_frags(st, ks + 1, (ks + 1) & 1);
        __builtin_amdgcn_sched_barrier(0);
        mfmas(ks & 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        lds_frags(st, ks, 0);
        mfmas(0);
      }
    }
    if constexpr (Cfg::STAGES == 2) {
      if (more) sstore(stage ^ 1, slab + 1);
      __syncthreads();
    } else {
      __syncthreads();
      if (more) sstore(0, slab + 1);
      __syncthreads();
    }
  }

  // Epilogue. acc[tn][tm][r] is output row m = m0 + wm*WM + tm*32 + lr, column
  // n = n0 + wn*WN + tn*32 + 8*(r/4) + 4*g + (r%4). Each wave passes its 32 x WN strip
  // through a private LDS patch (16-byte chunks XOR-swizzled by row) so that every store
  // instruction writes whole contiguous row segments. A lane keeps the same four columns
  // for every row of the strip (64 lanes cover 64/CH rows x CH chunks per step), so its
  // bias values are loaded once; IU steps are processed together so their LDS reads and
  // residual loads overlap, and the activation is selected once per group, not per element.
  constexpr int WN = Cfg::WN, CH = WN / 4, ITERS = (32 * CH) / 64, RSTEP = 64 / CH;
  constexpr int IU = ITERS < 4 ? ITERS : 4;
  float* sC = reinterpret_cast<float*>(smem) + wave * (32 * WN);
  const int ec = lane % CH, er = lane / CH;
  const int n = n0 + wn * WN + ec * 4;
  const bool n_ok = n < a.N;
  const bool full = a.vec_ok && (n + 3 < a.N) && !(n < a.nsplit && n + 3 >= a.nsplit);
  float bias4[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.bias && n_ok) {
#pragma unroll
    for (int e = 0; e < 4; ++e) if (n + e < a.N) bias4[e] = a.bias[n + e];
  }
  const bool res_f32 = a.res_dtype == DT_F32, res_f16 = a.res_dtype == DT_F16;
  const float descale = a.descale, alpha = a.alpha;
  float local_amax = 0.f;

  static_for<0, TM>([&](auto tmc) {
    constexpr int tm = decltype(tmc)::value;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int chunk = tn * 8 + 2 * rq + g;
        f32x4_t v4 = {acc[tn][tm][4 * rq], acc[tn][tm][4 * rq + 1], acc[tn][tm][4 * rq + 2], acc[tn][tm][4 * rq + 3]};
        *reinterpret_cast<f32x4_t*>(sC + lr * WN + ((chunk ^ (lr & (CH - 1))) << 2)) = v4;
      }
    wave_lds_fence();
#pragma unroll 1
    for (int ito = 0; ito < ITERS; ito += IU) {
      const int rbase = er + ito * RSTEP;
      const int mbase = m0 + wm * Cfg::WM + tm * 32 + rbase;
      float v[IU][4];
      f32x4_t lv[IU];
#pragma unroll
      for (int it = 0; it < IU; ++it) {
        const int r = rbase + it * RSTEP;
        lv[it] = *reinterpret_cast<const f32x4_t*>(sC + r * WN + ((ec ^ (r & (CH - 1))) << 2));
      }
      float rv[IU][4];
      if (a.res) {
#pragma unroll
        for (int it = 0; it < IU; ++it) {
          const int m = mbase + it * RSTEP;
#pragma unroll
          for (int e = 0; e < 4; ++e) rv[it][e] = 0.f;
          if (m < a.M && n_ok) {
            const long ro = (long)(a.res_rows > 0 ? m % a.res_rows : m) * a.ldr + n;
            if (res_f32) {
              const float* rp = reinterpret_cast<const float*>(a.res) + ro;
              if (full) { const float4 r4 = *reinterpret_cast<const float4*>(rp); rv[it][0] = r4.x; rv[it][1] = r4.y; rv[it][2] = r4.z; rv[it][3] = r4.w; }
              else {
#pragma unroll
                for (int e = 0; e < 4; ++e) if (n + e < a.N) rv[it][e] = rp[e];
              }
            } else {
              const uint16_t* rp = reinterpret_cast<const uint16_t*>(a.res) + ro;
              uint16_t rb[4] = {0, 0, 0, 0};
              if (full) {
                const uint2 r2 = *reinterpret_cast<const uint2*>(rp);
                rb[0] = (uint16_t)(r2.x & 0xffff); rb[1] = (uint16_t)(r2.x >> 16);
                rb[2] = (uint16_t)(r2.y & 0xffff); rb[3] = (uint16_t)(r2.y >> 16);
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) if (n + e < a.N) rb[e] = rp[e];
              }
#pragma unroll
              for (int e = 0; e < 4; ++e) rv[it][e] = res_f16 ? f16_bits_to_f32(rb[e]) : bf16_bits_to_f32(rb[e]);
            }
          }
        }
      }
#pragma unroll
      for (int it = 0; it < IU; ++it)
#pragma unroll
        for (int e = 0; e < 4; ++e) v[it][e] = fmaf(lv[it][e], descale, bias4[e]);
      switch (a.act) {  // uniform
        case ACT_GELU:
#pragma unroll
          for (int it = 0; it < IU; ++it)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[it][e] = act_gelu(v[it][e]);
          break;
        case ACT_MISH:
#pragma unroll
          for (int it = 0; it < IU; ++it)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[it][e] = act_mish(v[it][e]);
          break;
        case ACT_SWISH:
#pragma unroll
          for (int it = 0; it < IU; ++it)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[it][e] = act_swish(v[it][e]);
          break;
        default: break;
      }
      if (a.res) {
#pragma unroll
        for (int it = 0; it < IU; ++it)
#pragma unroll
          for (int e = 0; e < 4; ++e) v[it][e] = fmaf(v[it][e], alpha, rv[it][e]);
      } else {
#pragma unroll
        for (int it = 0; it < IU; ++it)
#pragma unroll
          for (int e = 0; e < 4; ++e) v[it][e] *= alpha;
      }
      if (a.amax) {
#pragma unroll
        for (int it = 0; it < IU; ++it)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (mbase + it * RSTEP < a.M && n + e < a.N) local_amax = fmaxf(local_amax, fabsf(v[it][e]));
      }
      if constexpr (OUT_DT == DT_FP8) {
        const float os = a.out_scale;
#pragma unroll
        for (int it = 0; it < IU; ++it)
#pragma unroll
          for (int e = 0; e < 4; ++e) v[it][e] *= os;
      }
#pragma unroll
      for (int it = 0; it < IU; ++it) {
        const int m = mbase + it * RSTEP;
        if (m >= a.M || !n_ok) continue;
        if (full) {
          if (n < a.nsplit) store4<OUT_DT>(a.C, (long)m * a.ldc + n, v[it]);
          else store4<OUT_DT>(a.C2, (long)m * a.ldc2 + (n - a.nsplit), v[it]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e >= a.N) continue;
            if (n + e < a.nsplit) store1<OUT_DT>(a.C, (long)m * a.ldc + n + e, v[it][e]);
            else store1<OUT_DT>(a.C2, (long)m * a.ldc2 + (n + e - a.nsplit), v[it][e]);
          }
        }
      }
    }
    wave_lds_fence();
  });
  if (a.amax) {
    local_amax = wave_max(local_amax);
    if (lane == 0) atomic_amax(a.amax, local_amax);
  }
}

// ---- host-side dispatch -------------------------------------------------------------
//                 BM   BN  WGM WGN stages frag_db min_waves
// Measured on MI355X (M=65536, K=1024..8192): the 8-wave 256x256 tile (two waves per SIMD
// covering each other's LDS and barrier stalls) beats the 4-wave 256x256 tile with
// double-buffered fragments, the single-stage 256x128 tile and the 128x128 tile for
// every trunk shape in both fp8 and bf16.
typedef GemmCfg<256, 256, 2, 4, 2, 0, 2> CfgBig;    // 8 waves, 128x64 per wave, two waves per SIMD
typedef GemmCfg<128, 128, 2, 2, 2, 0, 2> CfgMid;    // 4 waves, 64x64 per wave, two workgroups per CU
typedef GemmCfg<64, 64, 2, 2, 2, 0, 2> CfgSmall;    // 4 waves, 32x32 per wave

template <typename Cfg, int IN_DT, int OUT_DT>
static hipError_t launch_cfg(const GemmArgs& a, hipStream_t st) {
  static bool attr_set[16] = {};
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_kernel<Cfg, IN_DT, OUT_DT>;
  if (dev >= 0 && dev < 16 && !attr_set[dev]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(Cfg::NT), Cfg::LDS_BYTES, st, a);
  return hipGetLastError();
}

template <int IN_DT, int OUT_DT>
static hipError_t launch_in_out(const GemmArgs& a, int tile, hipStream_t st) {
  if (tile == 0) {
    // Largest tile that still gives every CU a workgroup.
    const long big = (long)((a.M + 255) / 256) * ((a.N + 255) / 256);
    const long mid = (long)((a.M + 127) / 128) * ((a.N + 127) / 128);
    tile = big >= 256 ? 3 : mid >= 256 ? 2 : 1;
  }
  if (tile == 3) return launch_cfg<CfgBig, IN_DT, OUT_DT>(a, st);
  if (tile == 2) return launch_cfg<CfgMid, IN_DT, OUT_DT>(a, st);
  return launch_cfg<CfgSmall, IN_DT, OUT_DT>(a, st);
}

template <int IN_DT>
static hipError_t launch_in(const GemmArgs& a, int out_dt, int tile, hipStream_t st) {
  switch (out_dt) {
    case DT_F32: return launch_in_out<IN_DT, DT_F32>(a, tile, st);
    case DT_BF16: return launch_in_out<IN_DT, DT_BF16>(a, tile, st);
    case DT_F16: return launch_in_out<IN_DT, DT_F16>(a, tile, st);
    case DT_FP8: return launch_in_out<IN_DT, DT_FP8>(a, tile, st);
  }
  return hipErrorInvalidValue;
}

// in_dt: element type of A and W; out_dt: element type of C/C2; tile: 0 auto, 1 = 64x64,
// 2 = 128x128, 3 = 256x256 workgroup tile.
hipError_t launch_gemm(GemmArgs a, int in_dt, int out_dt, int tile, hipStream_t st) {
  if (a.M <= 0 || a.N <= 0) return hipSuccess;
  const int esz = in_dt == DT_FP8 ? 1 : 2;
  // 16-byte global loads along K: rows must start 16-byte aligned and K must be a
  // whole number of 16-byte chunks.
  if (((long)a.K * esz) % 16 || (a.lda * esz) % 16 || (a.ldw * esz) % 16 ||
      (reinterpret_cast<uintptr_t>(a.A) & 15) || (reinterpret_cast<uintptr_t>(a.W) & 15))
    return hipErrorInvalidValue;
  if (a.nsplit <= 0 || a.nsplit > a.N || !a.C2) { a.nsplit = a.N; a.C2 = a.C; a.ldc2 = a.ldc; }
  const int osz = dtype_size(out_dt);
  const int w = 4;  // elements per vector access
  bool ok = (a.ldc % w == 0) && (reinterpret_cast<uintptr_t>(a.C) % (osz * w) == 0) &&
            (a.ldc2 % w == 0) && (reinterpret_cast<uintptr_t>(a.C2) % (osz * w) == 0) && (a.nsplit % w == 0 || a.nsplit == a.N);
  if (a.res) {
    const int rsz = dtype_size(a.res_dtype);
    ok = ok && (a.ldr % w == 0) && (reinterpret_cast<uintptr_t>(a.res) % (rsz * w) == 0);
  }
  a.vec_ok = ok ? 1 : 0;
  switch (in_dt) {
    case DT_BF16: return launch_in<DT_BF16>(a, out_dt, tile, st);
    case DT_F16: return launch_in<DT_F16>(a, out_dt, tile, st);
    case DT_FP8: return launch_in<DT_FP8>(a, out_dt, tile, st);
  }
  return hipErrorInvalidValue;
}

}  // namespace crl
