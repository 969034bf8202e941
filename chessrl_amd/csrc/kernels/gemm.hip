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
#include <mutex>
#include <type_traits>
#include <unordered_map>

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

// NT: store with the non-temporal hint, so a streamed output does not evict the operands from L2.
template <int OUT_DT, int NT = 0>
__device__ __forceinline__ void store8(void* base, long off, const float v[8]) {
  auto put = [](i32x4_t* p, i32x4_t x) {
    if constexpr (NT) __builtin_nontemporal_store(x, p);
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
    if constexpr (NT) __builtin_nontemporal_store(x, p);
    else *p = x;
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
template <int WM, int WN, int OUT_DT>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& a, f32x16_t (&acc)[WN / 32][WM / 32], float* sC, int mw0, int nw0, int lane) {
  constexpr int TM = WM / 32, TN = WN / 32, CH4 = WN / 4, CP = WN / 8, RSTEP = 64 / CP, ITERS = 32 / RSTEP;
  const int lr = lane & 31, g = lane >> 5;
  const int ec = lane % CP, er = lane / CP;
  const int n = nw0 + ec * 8;
  const bool n_ok = n < a.N;
  const bool full = a.vec_ok && (n + 7 < a.N) && ((n < a.nsplit) == (n + 7 < a.nsplit));
  float bias8[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) bias8[e] = (a.bias && n + e < a.N) ? a.bias[n + e] : 0.f;
  const int res_dt = a.res_dtype;
  const float descale = a.descale, alpha = a.alpha;
  float local_amax = 0.f;

  // Raw residual bits, 16 bytes per step and set. 16-bit residuals use the two sets as a double
  // buffer over strips; an fp32 residual (8 values = 32 bytes) uses both sets for the current
  // strip (low and high half), i.e. it is fetched at the start of its own strip.
  const bool res32 = res_dt == DT_F32;
  uint4 rraw[2][ITERS];
  auto load_res = [&](int tm, int set, int half) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int m = mw0 + tm * 32 + er + it * RSTEP;
      uint4 val = make_uint4(0, 0, 0, 0);
      if (m < a.M && n_ok) {
        const long ro = (long)(a.res_rows > 0 ? m % a.res_rows : m) * a.ldr + n;
        if (res32) {
          const float* rp = reinterpret_cast<const float*>(a.res) + ro + 4 * half;
          if (full) val = *reinterpret_cast<const uint4*>(rp);
          else {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (n + 4 * half + e < a.N) ? __float_as_uint(rp[e]) : 0u;
            val = make_uint4(w[0], w[1], w[2], w[3]);
          }
        } else {
          const uint16_t* rp = reinterpret_cast<const uint16_t*>(a.res) + ro;
          if (full) val = *reinterpret_cast<const uint4*>(rp);
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
  auto res_value = [&](int tm, int it, int e) -> float {
    if (res32) {
      const uint4 q = rraw[e >> 2][it];
      const uint32_t w[4] = {q.x, q.y, q.z, q.w};
      return __uint_as_float(w[e & 3]);
    }
    const uint4 q = rraw[tm & 1][it];
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    const uint16_t h = (uint16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffff));
    return res_dt == DT_F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
  };

  if (a.res && !res32) load_res(0, 0, 0);
  static_for<0, TM>([&](auto tmc) {
    constexpr int tm = decltype(tmc)::value;
    if (a.res) {
      if (res32) { load_res(tm, 0, 0); load_res(tm, 1, 1); }
      else if constexpr (tm + 1 < TM) load_res(tm + 1, (tm + 1) & 1, 0);
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int chunk = tn * 8 + 2 * rq + g;
        f32x4_t v4 = {acc[tn][tm][4 * rq], acc[tn][tm][4 * rq + 1], acc[tn][tm][4 * rq + 2], acc[tn][tm][4 * rq + 3]};
        *reinterpret_cast<f32x4_t*>(sC + lr * WN + ((chunk ^ (lr & (CH4 - 1))) << 2)) = v4;
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
    }
    switch (a.act) {  // uniform
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
    if (a.res) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[it][e] = fmaf(v[it][e], alpha, res_value(tm, it, e));
    } else {
#pragma unroll
      for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[it][e] *= alpha;
    }
    if (a.amax) {
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
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int m = mw0 + tm * 32 + er + it * RSTEP;
      if (m >= a.M || !n_ok) continue;
      if (full) {
        void* dst = n < a.nsplit ? a.C : a.C2;
        const long off = n < a.nsplit ? (long)m * a.ldc + n : (long)m * a.ldc2 + (n - a.nsplit);
        if (a.stream_out) store8<OUT_DT, 1>(dst, off, v[it]);
        else store8<OUT_DT, 0>(dst, off, v[it]);
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
  if (a.amax) {
    local_amax = wave_max(local_amax);
    if (lane == 0) atomic_amax(a.amax, local_amax);
  }
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
  int slice = 0;
  if (a.k_slices > 1) { slice = pid % a.k_slices; pid /= a.k_slices; }
  const int tile_m = pid / tiles_n, tile_n = pid - tile_m * tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const long kbytes = (long)a.K * ESZ;
  const int nslab_all = (int)((kbytes + 127) >> 7);
  // A K-sliced launch walks only this workgroup's slabs and leaves the raw fp32 sums in its own copy of C.
  const int slab0 = a.k_slices > 1 ? slice * a.slabs_per_slice : 0;
  const int nslab = a.k_slices > 1 ? min(nslab_all, slab0 + a.slabs_per_slice) : nslab_all;
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

  gload(slab0);
  sstore(0, slab0);
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

  for (int slab = slab0; slab < nslab; ++slab) {
    const int stage = Cfg::STAGES == 2 ? ((slab - slab0) & 1) : 0;
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

  if (a.k_slices > 1) {
    GemmArgs b = a;
    b.C = b.C2 = reinterpret_cast<char*>(a.C) + (size_t)slice * a.M * a.ldc * dtype_size(OUT_DT);
    gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT>(b, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                           m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane);
    return;
  }
  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                         m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane);
}

// ---- second pass of a K-sliced GEMM -------------------------------------------------------------
// partial [ks, M, ldp] holds the raw fp32 sums of the slices. One thread per output row and group of four columns
// adds them in slice order (so the result does not depend on which workgroup finished first) and applies the
// epilogue of the one-pass kernels: C = res + alpha*act(descale*sum + bias), amax, the fp8 output scale, the C/C2 split.
template <int OUT_DT>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const GemmArgs a, const float* partial, int ks, long ldp) {
  const int groups = (a.N + 3) / 4;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const int m = (int)(idx / groups), n = (int)(idx - (long)m * groups) * 4;
  float local_amax = 0.f;
  if (m < a.M) {
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    const float* pp = partial + (long)m * ldp + n;
    for (int s = 0; s < ks; ++s) acc += *reinterpret_cast<const f32x4_t*>(pp + (long)s * a.M * ldp);   // ldp is a multiple of 4 and >= N rounded up
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float b = (a.bias && n + i < a.N) ? a.bias[n + i] : 0.f;
      v[i] = apply_act(fmaf(acc[i], a.descale, b), a.act);
    }
    if (a.res) {
      const long ro = (long)(a.res_rows > 0 ? m % a.res_rows : m) * a.ldr + n;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float rv = 0.f;
        if (n + i < a.N) {
          if (a.res_dtype == DT_F32) rv = reinterpret_cast<const float*>(a.res)[ro + i];
          else {
            const uint16_t h = reinterpret_cast<const uint16_t*>(a.res)[ro + i];
            rv = a.res_dtype == DT_F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
          }
        }
        v[i] = fmaf(v[i], a.alpha, rv);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= a.alpha;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (n + i >= a.N) continue;
      local_amax = fmaxf(local_amax, fabsf(v[i]));
      const float o = OUT_DT == DT_FP8 ? v[i] * a.out_scale : v[i];
      if (n + i < a.nsplit) store1<OUT_DT>(a.C, (long)m * a.ldc + n + i, o);
      else store1<OUT_DT>(a.C2, (long)m * a.ldc2 + (n + i - a.nsplit), o);
    }
  }
  if (a.amax) {
    local_amax = wave_max(local_amax);
    if ((threadIdx.x & 63) == 0) atomic_amax(a.amax, local_amax);
  }
}

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
  static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES > EPI_BYTES ? NSTAGE * STAGE_BYTES : EPI_BYTES;
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

template <typename Cfg, int IN_DT, int OUT_DT>
__global__ void __launch_bounds__(Cfg::NT, 2) gemm_dma_kernel(const GemmArgs a, const uint8_t* zeros) {
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
  // Inside an XCD's range the tiles are walked in groups of 8 x 4 (M x N), so the 32 workgroups resident on the
  // XCD share 8 activation tiles and 4 weight tiles (3 MB of operands at K = 1024 bytes, inside its 4 MB L2).
  int tile_m = pid / tiles_n, tile_n = pid - tile_m * tiles_n;
  {
    constexpr int GM = 8, GN = 4;
    const int tiles_m = (a.M + BM - 1) / BM;
    if (tiles_m % GM == 0 && tiles_n % GN == 0) {
      const int sr = pid / (GM * tiles_n), rem = pid - sr * (GM * tiles_n);
      const int ng = rem / (GM * GN), r2 = rem - ng * (GM * GN);
      tile_m = sr * GM + r2 / GN;
      tile_n = ng * GN + r2 % GN;
    }
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const long kbytes = (long)a.K * ESZ;
  const int nslab = (int)((kbytes + Cfg::ROWB - 1) / Cfg::ROWB);
  const long kmax = kbytes - 16;

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

#pragma unroll
  for (int s0 = 0; s0 < NSTAGE - 1; ++s0)
    if (s0 < nslab) issue(s0);

  for (int slab = 0; slab < nslab; ++slab) {
    // Loads still allowed in flight behind this slab's: LOADS per later slab already issued.
    const int ahead = nslab - 1 - slab;
    if (NSTAGE >= 4 && ahead >= 2) wait_vmcnt<2 * LOADS>();
    else if (NSTAGE >= 3 && ahead == 1) wait_vmcnt<LOADS>();
    else wait_vmcnt<0>();
    __syncthreads();
    if (slab + NSTAGE - 1 < nslab) issue(slab + NSTAGE - 1);
    const uint8_t* st = smem + (slab % NSTAGE) * Cfg::STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      Frag<IN_DT> wf[TN], xf[TM];
      read_frags(wf, xf, st, ks);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = mfma_frag<IN_DT>(wf[tn], xf[tm], acc[tn][tm]);
    }
  }

  __syncthreads();  // every wave is done with the ring before it becomes epilogue scratch

  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                         m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane);
}

// ---- host-side dispatch -------------------------------------------------------------
//                 BM   BN  WGM WGN stages frag_db min_waves
// Measured on MI355X (M=65536, N=1024..3072, K=1024..8192, fp8 and bf16, same job): the 256x256
// tile fed by direct-to-LDS loads with 128-byte rows and two stages (DmaCfg2) is 10-20 % faster
// than the same 8-wave tile with register staging; the 4-wave 256x256 tile (one wave per SIMD,
// with or without double-buffered fragments), a 256x128 single-stage tile at two workgroups per
// CU, a 4-stage ring of 64-byte rows (twice the barriers) and a persistent
// one-workgroup-per-CU loop (epilogue stores of tile t delay the first slab of tile t+1 because
// loads and stores share vmcnt) were all slower. The register-staged kernel serves the small tiles.
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

// One 256-byte block of zeros per device: the source of K-tail chunks for the direct-to-LDS loads.
static const uint8_t* device_zeros(hipError_t* err) {
  static uint8_t* z[16] = {};
  int dev = 0;
  *err = hipGetDevice(&dev);
  if (*err != hipSuccess || dev < 0 || dev >= 16) { if (*err == hipSuccess) *err = hipErrorInvalidDevice; return nullptr; }
  if (!z[dev]) {
    uint8_t* p = nullptr;
    *err = hipMalloc((void**)&p, 256);
    if (*err != hipSuccess) return nullptr;
    *err = hipMemset(p, 0, 256);
    if (*err != hipSuccess) { (void)hipFree(p); return nullptr; }
    z[dev] = p;
  }
  return z[dev];
}

template <typename DCfg, int IN_DT, int OUT_DT>
static hipError_t launch_dma(const GemmArgs& a, hipStream_t st) {
  static bool attr_set[16] = {};
  hipError_t e = hipSuccess;
  const uint8_t* zeros = device_zeros(&e);
  if (!zeros) return e;
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_dma_kernel<DCfg, IN_DT, OUT_DT>;
  if (!attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, DCfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + DCfg::BM - 1) / DCfg::BM) * ((a.N + DCfg::BN - 1) / DCfg::BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(DCfg::NT), DCfg::LDS_BYTES, st, a, zeros);
  return hipGetLastError();
}

// Workspace of the K-sliced GEMMs: one per (device, stream a launch is issued or recorded on), so launches that may
// run at the same time never share one. Lives until the process ends.
constexpr size_t SPLITK_WS_BYTES = 16u << 20;
static std::mutex g_ws_mutex;
static std::unordered_map<uint64_t, float*> g_ws;
static hipError_t workspace_for(hipStream_t st, float** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t key = (reinterpret_cast<uint64_t>(st) << 4) ^ (uint64_t)(dev & 15);
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto it = g_ws.find(key);
  if (it != g_ws.end()) { *out = it->second; return hipSuccess; }
  float* p = nullptr;
  e = hipMalloc((void**)&p, SPLITK_WS_BYTES);
  if (e != hipSuccess) return e;
  g_ws.emplace(key, p);
  *out = p;
  return hipSuccess;
}
hipError_t gemm_prepare_stream(hipStream_t st) {
  float* p = nullptr;
  return workspace_for(st, &p);
}

// Few output tiles and a long K leave most CUs idle while a few walk K alone (M=128, N=768, K=3072: 24 workgroups
// of 48 slabs each). Then K is cut into slices, one workgroup per (tile, slice) writes its raw sums, and a second
// small kernel adds the slices and applies the epilogue. Returns the number of slices (1: not worth it / no room).
static int splitk_plan(const GemmArgs& a, int esz, bool forced, int* slabs_per_slice) {
  const long tiles = (long)((a.M + 63) / 64) * ((a.N + 63) / 64);
  const int nslab = (int)(((long)a.K * esz + 127) >> 7);
  if (!forced && (tiles > 64 || nslab < 16)) return 1;
  int ks = (int)std::min<long>(std::max(nslab / 4, 1), (256 + tiles - 1) / tiles);
  if (forced) ks = std::max(ks, std::min(nslab, 2));
  const int per = (nslab + ks - 1) / ks;
  ks = (nslab + per - 1) / per;
  const long ldp = (a.N + 7) / 8 * 8;
  if (ks < 2 || (size_t)ks * a.M * ldp * sizeof(float) > SPLITK_WS_BYTES) return 1;
  *slabs_per_slice = per;
  return ks;
}

template <int IN_DT, int OUT_DT>
static hipError_t launch_splitk(const GemmArgs& a, int ks, int per, hipStream_t st) {
  float* ws = nullptr;
  hipError_t e = workspace_for(st, &ws);
  if (e != hipSuccess) return e;
  const long ldp = (a.N + 7) / 8 * 8;
  GemmArgs b = a;
  b.C = b.C2 = ws; b.ldc = b.ldc2 = ldp; b.nsplit = a.N;
  b.bias = nullptr; b.res = nullptr; b.amax = nullptr; b.act = ACT_NONE; b.descale = 1.f; b.alpha = 1.f; b.out_scale = 1.f;
  b.vec_ok = 1; b.stream_out = 0; b.k_slices = ks; b.slabs_per_slice = per;
  static bool attr_set[16] = {};
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_kernel<CfgSmall, IN_DT, DT_F32>;
  if (dev >= 0 && dev < 16 && !attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, CfgSmall::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + 63) / 64) * ((a.N + 63) / 64);
  hipLaunchKernelGGL(kern, dim3(tiles * ks), dim3(CfgSmall::NT), CfgSmall::LDS_BYTES, st, b);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  const long threads = (long)a.M * ((a.N + 3) / 4);
  hipLaunchKernelGGL((splitk_reduce_kernel<OUT_DT>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, a, ws, ks, ldp);
  return hipGetLastError();
}

template <int IN_DT, int OUT_DT>
static hipError_t launch_in_out(const GemmArgs& a, int tile, hipStream_t st) {
  if (tile == 0 || tile == 4) {
    int per = 0;
    const int ks = splitk_plan(a, IN_DT == DT_FP8 ? 1 : 2, tile == 4, &per);
    if (ks > 1) return launch_splitk<IN_DT, OUT_DT>(a, ks, per, st);
    if (tile == 4) tile = 1;
  }
  if (tile == 0) {
    // Largest tile that still gives every CU a workgroup.
    const long big = (long)((a.M + 255) / 256) * ((a.N + 255) / 256);
    const long mid = (long)((a.M + 127) / 128) * ((a.N + 127) / 128);
    tile = big >= 256 ? 3 : mid >= 256 ? 2 : 1;
  }
  if (tile == 3) return launch_dma<DmaCfg2, IN_DT, OUT_DT>(a, st);
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
// 2 = 128x128, 3 = 256x256 (direct-to-LDS loads), 4 = 64x64 tiles with K cut into slices.
hipError_t launch_gemm(GemmArgs a, int in_dt, int out_dt, int tile, hipStream_t st) {
  if (a.M <= 0 || a.N <= 0) return hipSuccess;
  const int esz = in_dt == DT_FP8 ? 1 : 2;
  // 16-byte global loads along K: rows must start 16-byte aligned and K must be a
  // whole number of 16-byte chunks.
  if (((long)a.K * esz) % 16 || (a.lda * esz) % 16 || (a.ldw * esz) % 16 ||
      (reinterpret_cast<uintptr_t>(a.A) & 15) || (reinterpret_cast<uintptr_t>(a.W) & 15))
    return hipErrorInvalidValue;
  if (a.nsplit <= 0 || a.nsplit > a.N || !a.C2) { a.nsplit = a.N; a.C2 = a.C; a.ldc2 = a.ldc; }
  // 8-element vector accesses along N: row strides in multiples of 8 elements, bases aligned to
  // 16 bytes (the fp32 paths use two 16-byte accesses).
  const int w = 8;
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  bool ok = (a.ldc % w == 0) && al16(a.C) && (a.ldc2 % w == 0) && al16(a.C2) && (a.nsplit % w == 0 || a.nsplit == a.N);
  if (out_dt == DT_FP8) ok = ok && (reinterpret_cast<uintptr_t>(a.C) & 7) == 0;
  if (a.res) ok = ok && (a.ldr % w == 0) && al16(a.res);
  a.vec_ok = ok ? 1 : 0;
  // An output beyond the 32 MB of L2 (8 XCDs x 4 MB) cannot be kept for the consumer anyway: stream it past the
  // caches so it does not push the operand tiles out (measured +6..10 % on the 0.5-1.6 GB outputs of a 4096-position batch).
  a.stream_out = (long)a.M * a.N * dtype_size(out_dt) > (64L << 20) ? 1 : 0;
  switch (in_dt) {
    case DT_BF16: return launch_in<DT_BF16>(a, out_dt, tile, st);
    case DT_F16: return launch_in<DT_F16>(a, out_dt, tile, st);
    case DT_FP8: return launch_in<DT_FP8>(a, out_dt, tile, st);
  }
  return hipErrorInvalidValue;
}

}  // namespace crl
