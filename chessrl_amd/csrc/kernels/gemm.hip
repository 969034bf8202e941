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
#include <atomic>
#include <mutex>
#include <unordered_map>

#include "gemm_tile.hpp"

namespace crl {

// KG_ > 1: KG_ groups of WGM x WGN waves share one output tile and take the K slabs in turn (group g the slabs
// g, g + KG, ...), each with its own LDS stages; their accumulators are added in group order at the end.
template <int BM_, int BN_, int WGM_, int WGN_, int STAGES_, int FRAG_DB_, int MIN_WAVES_, int KG_ = 1>
struct GemmCfg {
  static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_, STAGES = STAGES_, FRAG_DB = FRAG_DB_;
  static constexpr int MIN_WAVES = MIN_WAVES_, KG = KG_;
  static constexpr int NW = WGM * WGN, NT = 64 * NW;        // waves and threads of one group
  static constexpr int NT_ALL = NT * KG;
  static constexpr int WM = BM / WGM, WN = BN / WGN;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int ROWS_PER_PASS = NT / 8;
  static constexpr int A_PASSES = BM / ROWS_PER_PASS, W_PASSES = BN / ROWS_PER_PASS;
  static constexpr int STAGE_BYTES = (BM + BN) * 128;
  static constexpr int EPI_BYTES = NW * 32 * WN * 4;
  static constexpr int GROUP_BYTES = STAGES * STAGE_BYTES > EPI_BYTES ? STAGES * STAGE_BYTES : EPI_BYTES;
  static constexpr int LDS_BYTES = GROUP_BYTES * KG;
  static_assert(KG == 1 || BM * BN * 4 <= GROUP_BYTES, "a group's accumulators must fit its own LDS region");
  static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile/threads mismatch");
  static_assert(WN >= 32 && WM >= 32, "wave tile too small");
};

template <typename Cfg, int IN_DT, int OUT_DT, int RES_NORM = 0>
__global__ void __launch_bounds__(Cfg::NT_ALL, Cfg::MIN_WAVES) gemm_kernel(const GemmArgs a) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, KG = Cfg::KG;
  constexpr int ESZ = (IN_DT == DT_FP8) ? 1 : 2;
  constexpr int KSTEPS = (IN_DT == DT_FP8) ? 2 : 4;
  extern __shared__ __align__(16) uint8_t smem_all[];

  const int kg = KG > 1 ? (int)threadIdx.x / Cfg::NT : 0;          // wave-uniform
  uint8_t* smem = smem_all + kg * Cfg::GROUP_BYTES;
  const int tid = KG > 1 ? (int)threadIdx.x - kg * Cfg::NT : (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
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
    const bool kok = slab < nslab && ((long)slab << 7) + kmine <= kmax;   // a group's turn may fall past the last slab
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

  gload(slab0 + kg);
  sstore(0, slab0 + kg);
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

  // Every group runs the same number of rounds (the barriers are workgroup-wide); a turn past the last slab works on zeros.
  for (int slab = slab0 + kg, round = 0; slab - kg < nslab; slab += KG, ++round) {
    const int stage = Cfg::STAGES == 2 ? (round & 1) : 0;
    const uint8_t* st = smem + stage * Cfg::STAGE_BYTES;
    const bool more = slab - kg + KG < nslab;
    if (more) gload(slab + KG);
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
      if (more) sstore(stage ^ 1, slab + KG);
      __syncthreads();
    } else {
      __syncthreads();
      if (more) sstore(0, slab + KG);
      __syncthreads();
    }
  }

  if constexpr (KG > 1) {
    // Groups 1.. leave their accumulators in their own LDS region (its stages are dead after the last barrier);
    // group 0 adds them in group order and alone runs the epilogue.
    float* mine = reinterpret_cast<float*>(smem) + (wave * 64 + lane) * (TN * TM * 16);
    if (kg > 0) {
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4)
            *reinterpret_cast<f32x4_t*>(mine + (i * TM + j) * 16 + 4 * r4) =
                f32x4_t{acc[i][j][4 * r4], acc[i][j][4 * r4 + 1], acc[i][j][4 * r4 + 2], acc[i][j][4 * r4 + 3]};
    }
    __syncthreads();
    if (kg > 0) return;
#pragma unroll
    for (int gsrc = 1; gsrc < KG; ++gsrc) {
      const float* theirs = reinterpret_cast<const float*>(smem_all + gsrc * Cfg::GROUP_BYTES) + (wave * 64 + lane) * (TN * TM * 16);
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const f32x4_t t = *reinterpret_cast<const f32x4_t*>(theirs + (i * TM + j) * 16 + 4 * r4);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][4 * r4 + e] += t[e];
          }
    }
  }

  if (a.k_slices > 1) {
    GemmArgs b = a;
    b.C = b.C2 = reinterpret_cast<char*>(a.C) + (size_t)slice * a.M * a.ldc * dtype_size(OUT_DT);
    gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT>(b, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                             m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane);
    return;
  }
  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT, RES_NORM>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                                     m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane,
                                                     reinterpret_cast<float*>(smem + Cfg::EPI_BYTES) + wave * (2 * Cfg::WM));
}

// ---- second pass of a K-sliced GEMM -------------------------------------------------------------
// partial [ks, M, ldp] holds the raw fp32 sums of the slices. One thread per output row and group of four columns
// adds them in slice order (so the result does not depend on which workgroup finished first) and applies the
// epilogue of the one-pass kernels: C = res + alpha*act(descale*sum + bias), amax, the fp8 output scale, the C/C2 split.
// The four columns n..n+3 of row m: slices added in order, epilogue applied, result stored; v receives the values
// (as stored: rounded to the output type) and the return value their largest magnitude.
template <int OUT_DT>
__device__ __forceinline__ float reduce_columns4(const GemmArgs& a, const float* partial, int ks, long ldp, int m, int n, float (&v)[4]) {
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  const float* pp = partial + (long)m * ldp + n;
#pragma unroll 8
  for (int s = 0; s < ks; ++s) acc += *reinterpret_cast<const f32x4_t*>(pp + (long)s * a.M * ldp);   // ldp is a multiple of 4 and >= N rounded up
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
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (n + i >= a.N) { v[i] = 0.f; continue; }
    amax = fmaxf(amax, fabsf(v[i]));
    const float o = OUT_DT == DT_FP8 ? v[i] * a.out_scale : v[i];
    if (n + i < a.nsplit) store1<OUT_DT>(a.C, (long)m * a.ldc + n + i, o);
    else store1<OUT_DT>(a.C2, (long)m * a.ldc2 + (n + i - a.nsplit), o);
    if constexpr (OUT_DT == DT_BF16) v[i] = bf16_bits_to_f32(f32_to_bf16_bits(v[i]));
    else if constexpr (OUT_DT == DT_F16) v[i] = f16_bits_to_f32(f32_to_f16_bits(v[i]));
  }
  return amax;
}

template <int OUT_DT>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const GemmArgs a, const float* partial, int ks, long ldp) {
  const int groups = (a.N + 3) / 4;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const int m = (int)(idx / groups), n = (int)(idx - (long)m * groups) * 4;
  float local_amax = 0.f;
  if (m < a.M) {
    float v[4];
    local_amax = reduce_columns4<OUT_DT>(a, partial, ks, ldp, m, n, v);
  }
  if (a.amax) {
    local_amax = wave_max(local_amax);
    if ((threadIdx.x & 63) == 0) atomic_amax(a.amax, local_amax);
  }
}

// The same pass with the LayerNorm that follows the GEMM folded in (F.layer_norm over the N columns of the stored
// result, model_bis.py:34): one workgroup per row, up to 4096 columns, wave sums added in wave order. It takes one
// launch out of every such GEMM + norm pair of a token step, where a launch costs as much as the work.
template <int OUT_DT>
__global__ void __launch_bounds__(256) splitk_reduce_ln_kernel(const GemmArgs a, const float* partial, int ks, long ldp) {
  __shared__ float s_red[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = blockIdx.x;
  float v[4][4];
  float local_amax = 0.f, s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = (i * 256 + tid) * 4;
    if (n < a.N) {
      local_amax = fmaxf(local_amax, reduce_columns4<OUT_DT>(a, partial, ks, ldp, m, n, v[i]));
      s += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
    }
  }
  s = wave_sum(s);
  if (lane == 0) s_red[0][wave] = s;
  __syncthreads();
  const float mean = a.ln_rms ? 0.f : (((s_red[0][0] + s_red[0][1]) + s_red[0][2]) + s_red[0][3]) / (float)a.N;
  const float* ln_beta = a.ln_rms ? nullptr : a.ln_beta;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = (i * 256 + tid) * 4;
    if (n < a.N) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < a.N) { const float d = v[i][e] - mean; q += d * d; }
    }
  }
  q = wave_sum(q);
  if (lane == 0) s_red[1][wave] = q;
  __syncthreads();
  const float rstd = rsqrtf((((s_red[1][0] + s_red[1][1]) + s_red[1][2]) + s_red[1][3]) / (float)a.N + a.ln_eps);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = (i * 256 + tid) * 4;
    if (n < a.N) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (n + e >= a.N) continue;
        const float y = (v[i][e] - mean) * rstd * a.ln_gamma[n + e] + (ln_beta ? ln_beta[n + e] : 0.f);
        const long off = (long)m * a.ln_ldo + n + e;
        if (a.ln_out_dtype == DT_F32) reinterpret_cast<float*>(a.ln_out)[off] = y;
        else reinterpret_cast<uint16_t*>(a.ln_out)[off] = a.ln_out_dtype == DT_BF16 ? f32_to_bf16_bits(y) : f32_to_f16_bits(y);
      }
    }
  }
  if (a.amax) {
    local_amax = wave_max(local_amax);
    if (lane == 0) atomic_amax(a.amax, local_amax);
  }
}

// ---- host-side dispatch -------------------------------------------------------------
//                 BM   BN  WGM WGN stages frag_db min_waves
// Measured on MI355X (M=65536, N=1024..3072, K=1024..8192, fp8 and bf16, same job): the 256x256
// tile fed by direct-to-LDS loads with 128-byte rows and two stages (DmaCfg2) is 10-20 % faster
// than the same 8-wave tile with register staging; a 256x128 single-stage tile at two workgroups per
// CU, a 4-stage ring of 64-byte rows (twice the barriers) and a one-workgroup-per-CU loop over several
// tiles (with bare barriers and a counted wait past the previous tile's stores too) were slower or equal.
// The register-staged kernel serves the small tiles.
typedef GemmCfg<128, 128, 2, 2, 2, 0, 2> CfgMid;    // 4 waves, 64x64 per wave, two workgroups per CU
typedef GemmCfg<64, 64, 2, 2, 2, 0, 2> CfgSmall;    // 4 waves, 32x32 per wave
typedef GemmCfg<64, 64, 2, 2, 2, 0, 2, 4> CfgSmallK4;   // the same tile walked by 4 groups of 4 waves, K slabs in turn

// Compute units of the current device (0 if the query fails: callers then take their conservative branch).
static int device_cus() {
  static std::atomic<int> cus[16] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 0;
  int n = cus[dev];
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cus[dev] = n;
  }
  return n;
}

template <typename Cfg, int IN_DT, int OUT_DT, int RES_NORM = 0>
static hipError_t launch_cfg(const GemmArgs& a, hipStream_t st) {
  if constexpr (!RES_NORM) {
    if (a.res_stats) {
      // The residual-normalising epilogue exists for the case that uses it (e4m3 operands, bf16 output and residual),
      // on every tile size, so that a row's result does not depend on the tile its batch size selects.
      if constexpr (IN_DT == DT_FP8 && OUT_DT == DT_BF16 && Cfg::KG == 1) {
        if (!a.res || a.res_dtype != DT_BF16 || !a.res_gamma || a.res_rows > 0 || a.alpha == 0.f) return hipErrorInvalidValue;
        return launch_cfg<Cfg, IN_DT, OUT_DT, 1>(a, st);
      } else {
        return hipErrorInvalidValue;
      }
    }
  } else {
    static_assert(Cfg::EPI_BYTES + Cfg::NW * 2 * Cfg::WM * 4 <= Cfg::LDS_BYTES, "row statistics need room behind the epilogue patches");
  }
  static std::atomic<bool> attr_set[16] = {};
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_kernel<Cfg, IN_DT, OUT_DT, RES_NORM>;
  if (dev >= 0 && dev < 16 && !attr_set[dev]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(Cfg::NT_ALL), Cfg::LDS_BYTES, st, a);
  return hipGetLastError();
}

// Device memory the GEMM launchers keep outside any model: the block of zeros of the 256x256 kernel (one per device) and
// the workspaces of the K-sliced GEMMs issued through crl_gemm, one per (device, stream a launch is issued or recorded
// on) so that launches that may run at the same time never share one. release_gemm_globals() (crl_shutdown) frees them.
constexpr size_t SPLITK_WS_BYTES = 64u << 20;
static std::mutex g_ws_mutex;
static std::unordered_map<uint64_t, float*> g_ws;
static uint8_t* g_zeros[16] = {};
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

const uint8_t* device_zeros(hipError_t* err) {
  std::lock_guard<std::mutex> lock(g_ws_mutex);   // first calls on one device may come from several host threads
  int dev = 0;
  *err = hipGetDevice(&dev);
  if (*err != hipSuccess || dev < 0 || dev >= 16) { if (*err == hipSuccess) *err = hipErrorInvalidDevice; return nullptr; }
  if (!g_zeros[dev]) {
    uint8_t* p = nullptr;
    *err = hipMalloc((void**)&p, 256);
    if (*err != hipSuccess) return nullptr;
    *err = hipMemset(p, 0, 256);
    if (*err != hipSuccess) { (void)hipFree(p); return nullptr; }
    g_zeros[dev] = p;
  }
  return g_zeros[dev];
}

void release_gemm_globals() {
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  int cur = 0;
  const bool have_dev = hipGetDevice(&cur) == hipSuccess;
  for (auto& kv : g_ws) {
    if (have_dev) (void)hipSetDevice((int)(kv.first & 15));
    (void)hipFree(kv.second);
  }
  g_ws.clear();
  for (int d = 0; d < 16; ++d)
    if (g_zeros[d]) {
      if (have_dev) (void)hipSetDevice(d);
      (void)hipFree(g_zeros[d]);
      g_zeros[d] = nullptr;
    }
  if (have_dev) (void)hipSetDevice(cur);
}

// Few output tiles and a long K leave most CUs idle while a few walk K alone (M=128, N=768, K=3072: 24 workgroups
// of 48 slabs each). Then K is cut into slices, one workgroup per (tile, slice) writes its raw sums, and a second
// small kernel adds the slices and applies the epilogue. Returns the number of slices (1: not worth it / no room).
static int splitk_plan(const GemmArgs& a, int esz, bool forced, int* slabs_per_slice) {
  const long tiles = (long)((a.M + 63) / 64) * ((a.N + 63) / 64);
  const int nslab = (int)(((long)a.K * esz + 127) >> 7);
  // (a LayerNorm waiting to be folded into the second pass is worth the slices at half the K)
  if (!forced && (tiles > 64 || nslab < (a.ln_out ? 8 : 16))) return 1;
  int ks = (int)std::min<long>(std::min(std::max(nslab / 4, 1), 16), (256 + tiles - 1) / tiles);
  if (forced) ks = std::max(ks, std::min(nslab, 2));
  const int per = (nslab + ks - 1) / ks;
  ks = (nslab + per - 1) / per;
  const long ldp = (a.N + 7) / 8 * 8;
  if (ks < 2 || (size_t)ks * a.M * ldp * sizeof(float) > (a.splitk_ws ? (size_t)a.splitk_ws_bytes : SPLITK_WS_BYTES)) return 1;
  *slabs_per_slice = per;
  return ks;
}

// The same idea for the forward pass, where a row's result must not depend on how many rows the call has: narrow
// outputs with a very long K (the value head's 8192 -> 128 layer on one row per position: 128 slabs) are always cut
// into the same slices, a function of N and K alone, whenever the 64x64 tile is the choice (fewer than 256 tiles of
// 128x128, i.e. under 16384 rows at these widths; the workspace holds that case). At 64 rows that layer otherwise runs
// on two workgroups for 98 us. From 64 slabs on: at 32 (the bias generator's 2048 -> 256 layer) the ring kernels walk
// K in 10.3 us where the two passes of the sliced form take 11.3 (13.1 against 22.6 us at 4096 rows).
static int splitk_plan_fixed(const GemmArgs& a, int esz, int* slabs_per_slice) {
  const int nslab = (int)(((long)a.K * esz + 127) >> 7);
  if (a.N > 256 || nslab < 64) return 1;
  int ks = std::min(nslab / 16, 4);
  const int per = (nslab + ks - 1) / ks;
  ks = (nslab + per - 1) / per;
  const long ldp = (a.N + 7) / 8 * 8;
  if (ks < 2 || (size_t)ks * a.M * ldp * sizeof(float) > (a.splitk_ws ? (size_t)a.splitk_ws_bytes : SPLITK_WS_BYTES)) return 1;
  *slabs_per_slice = per;
  return ks;
}

bool gemm_folds_layernorm(const GemmArgs& a, int in_dt) {
  int per = 0;
  return a.k_parallel && a.N <= 4096 && (a.nsplit <= 0 || a.nsplit >= a.N || !a.C2) && splitk_plan(a, in_dt == DT_FP8 ? 1 : 2, false, &per) > 1;
}

template <typename Cfg, int IN_DT, int OUT_DT>
static hipError_t launch_splitk(const GemmArgs& a, int ks, int per, hipStream_t st) {
  if (a.res_stats) return hipErrorInvalidValue;   // the second pass adds the residual as stored: it has no normalising form
  float* ws = a.splitk_ws;
  hipError_t e = ws ? hipSuccess : workspace_for(st, &ws);
  if (e != hipSuccess) return e;
  const long ldp = (a.N + 7) / 8 * 8;
  GemmArgs b = a;
  b.C = b.C2 = ws; b.ldc = b.ldc2 = ldp; b.nsplit = a.N;
  b.bias = nullptr; b.res = nullptr; b.amax = nullptr; b.act = ACT_NONE; b.descale = 1.f; b.alpha = 1.f; b.out_scale = 1.f;
  b.vec_ok = 1; b.stream_out = 0; b.k_slices = ks; b.slabs_per_slice = per; b.splitk_ws = nullptr;
  static std::atomic<bool> attr_set[16] = {};
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_kernel<Cfg, IN_DT, DT_F32>;
  if (dev >= 0 && dev < 16 && !attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + 63) / 64) * ((a.N + 63) / 64);
  hipLaunchKernelGGL(kern, dim3(tiles * ks), dim3(Cfg::NT_ALL), Cfg::LDS_BYTES, st, b);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (a.ln_out) {
    hipLaunchKernelGGL((splitk_reduce_ln_kernel<OUT_DT>), dim3(a.M), dim3(256), 0, st, a, ws, ks, ldp);
    return hipGetLastError();
  }
  const long threads = (long)a.M * ((a.N + 3) / 4);
  hipLaunchKernelGGL((splitk_reduce_kernel<OUT_DT>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, a, ws, ks, ldp);
  return hipGetLastError();
}

template <int IN_DT, int OUT_DT>
static hipError_t launch_in_out(const GemmArgs& a, int tile, hipStream_t st) {
  if (a.ln_out && !gemm_folds_layernorm(a, IN_DT)) return hipErrorInvalidValue;   // only the K-sliced path has a whole row in one place
  if (a.res_stats && (a.k_parallel || (tile >= 4 && tile != 7 && tile != 9 && tile != 10 && tile != 12))) return hipErrorInvalidValue;   // the tiled kernels only
  // K = 256 e4m3 elements into a large 16-bit output (the attention-bias generator): the kernel whose workgroups keep
  // their rows of A and walk N (gemm_shortk_kernel.hpp; tile 13). It is the only one that writes the blocked layout, and
  // that is what it is for: M = 131072, N = 4096 takes 280 us through the 256x256 tile, 310 us here row-major and 191 us
  // here in blocks, so nothing picks it for a row-major output unasked.
  if (a.c_blocked || tile == 13) return launch_gemm_shortk(a, IN_DT, OUT_DT, st);
  if ((tile == 0 && a.k_parallel) || tile == 4) {
    int per = 0;
    const int ks = splitk_plan(a, IN_DT == DT_FP8 ? 1 : 2, tile == 4, &per);
    if (ks > 1) return launch_splitk<CfgSmall, IN_DT, OUT_DT>(a, ks, per, st);
    if (tile == 4) tile = 1;
  }
  if (tile == 0) {
    // Largest tile that still gives (nearly) every CU a workgroup. One round of 256x256 tiles takes about as long
    // whether 160 or 256 CUs have one (33-37 us at K=1024 in bf16), and from about 160 tiles on that is less than the
    // 128x128 tiles need (M=4096, N=3104: 47 -> 37 us; M=8192, N=1536: 39 -> 35 us; 128 tiles or fewer: slower).
    const long big = (long)((a.M + 255) / 256) * ((a.N + 255) / 256);
    const long mid = (long)((a.M + 127) / 128) * ((a.N + 127) / 128);
    tile = big >= 160 ? 3 : mid >= 256 ? 2 : 1;
    // Few 64x64 tiles: nothing else on the CU hides the latency of walking K slab by slab, so four groups of waves
    // share the walk (measured with weights coming from HBM, M=128, K=768: 9.8 -> 8.2 us at N=2304, 12.3 -> 9.0 us at
    // N=3072) where the ring kernels below, which hide it with slabs in flight, do not apply (M=128, K=768 from warm
    // caches: 7.1 us on four groups, 6.4 us on the ring; a 128-sequence rollout +4 %).
    const long small = (long)((a.M + 63) / 64) * ((a.N + 63) / 64);
    const long nslab = ((long)a.K * (IN_DT == DT_FP8 ? 1 : 2) + 127) >> 7;
    const bool ring_ok = !a.res_stats && ((long)a.K * (IN_DT == DT_FP8 ? 1 : 2)) % 128 == 0 && gemm_dmam_has(IN_DT, OUT_DT);
    if (tile == 1 && a.k_parallel && small <= 512 && nslab >= 8 && !(ring_ok && small <= device_cus())) tile = 5;
    // (a residual that is normalised on the fly needs the tiled kernels' epilogue: no K slices for it)
    if (tile == 1 && !a.k_parallel && !a.res_stats) {
      int per = 0;
      const int ks = splitk_plan_fixed(a, IN_DT == DT_FP8 ? 1 : 2, &per);
      if (ks > 1) return launch_splitk<CfgSmallK4, IN_DT, OUT_DT>(a, ks, per, st);
    }
    // Fewer than 256 tiles of 128x128 and K in whole slabs: the ring kernels of gemm_dmam_kernel.hpp (bit-equal). On 32x32
    // tiles while every such tile has a CU of its own (tile 16; one position), else on 64x64 tiles while every one of
    // those has (tile 15; M=64, N=1024, K=1024 bf16 with weights from HBM: 13.6 us register-staged, 8.4 us on 15; from
    // warm caches 9.1, 7.6 and, on 16, 6.9 us), on 128x128 tiles beyond (tile 11; M=1024, N=3104: 20.7 -> 14.9 us;
    // M=2048, N=1536: 18.0 -> 14.1 us; M=512, N=3104: 13.9 -> 12.5 us; level at M=1024, N=1536 and M=2048, N=1024).
    if (tile == 1 && ring_ok)
      tile = (long)((a.M + 31) / 32) * ((a.N + 31) / 32) <= device_cus() ? 16 : small <= device_cus() ? 15 : 11;
  }
  if (tile == 6 || tile == 8) return hipErrorInvalidValue;   // codes of two retired kernels
  // The 256x256 tile has three kernels. Eight waves in step (gemm_dma_kernel.hpp, tile 7): every operand type, any K. The
  // same with its address arithmetic out of the main loop (gemm_dmaf_kernel.hpp, tile 10): K in whole 128-byte slabs;
  // bit-equal and faster (the GEMMs of a 4096-position e4m3 forward: -4.9 %), so tile 3 means this one where it exists.
  // Four software-pipelined waves with 16x16x128 MFMAs (gemm_sp2_kernel.hpp, tile 9): e4m3, whole slabs; the faster main
  // loop (1.63 against 1.96 us per slab on random data) and the slower prologue and epilogue (10.0 against 7.7 us per
  // tile): it takes over from K = 4096 on.
  constexpr int ESZ = IN_DT == DT_FP8 ? 1 : 2;
  const bool slabs = (a.K * ESZ) % 128 == 0;
  if ((tile == 9 || tile == 10) && !slabs) tile = 7;
  if (tile == 3 && slabs) {
    if (IN_DT == DT_FP8 && OUT_DT != DT_F32 && a.K >= 4096 && !a.res_stats) tile = 9;
    else if (gemm_dmaf_has(IN_DT, OUT_DT, a.res_stats != nullptr) && (long)((a.M + 255) / 256) * ((a.N + 255) / 256) < 65536) tile = 10;
  }
  if (tile == 9) {
    if constexpr (IN_DT == DT_FP8 && OUT_DT != DT_F32) return launch_gemm_sp2(a, OUT_DT, st);
    else return hipErrorInvalidValue;
  }
  if (tile == 10) return gemm_dmaf_has(IN_DT, OUT_DT, a.res_stats != nullptr) ? launch_gemm_dmaf(a, IN_DT, OUT_DT, st) : hipErrorInvalidValue;
  if (tile == 3 || tile == 7) return launch_gemm_dma(a, IN_DT, OUT_DT, st);
  // The 128x128 tile has the register-staged kernel (any K, fp32 outputs, normalised residuals; two workgroups per CU;
  // tile 12 names it) and, for K in whole slabs, the direct-to-LDS kernel with three slabs in flight
  // (gemm_dmam_kernel.hpp, tile 11; bit-equal; one workgroup per CU). The second is 15 to 20 % faster while every tile has a
  // CU of its own (M=4096, N=1024, bf16: 20.1 -> 16.3 us at K=1024, 27.9 -> 23.0 at K=1536) and level beyond (384 tiles: 26.6 -> 24.9 us
  // from warm caches, 768 tiles: 48.1 -> 49.2 us; no difference inside a 64-position forward pass), so tile 2 picks it for
  // at most as many tiles as there are CUs.
  if (tile == 15 || tile == 16) return slabs && !a.res_stats && gemm_dmam_has(IN_DT, OUT_DT) ? launch_gemm_dmam(a, IN_DT, OUT_DT, st, tile == 16 ? 32 : 64) : hipErrorInvalidValue;
  if (tile == 11 && !slabs) tile = 12;
  if (tile == 2 || tile == 11) {
    const long mid_tiles = (long)((a.M + 127) / 128) * ((a.N + 127) / 128);
    const bool can = slabs && !a.res_stats && gemm_dmam_has(IN_DT, OUT_DT) && mid_tiles < 65536;
    if (can && (tile == 11 || mid_tiles <= device_cus())) return launch_gemm_dmam(a, IN_DT, OUT_DT, st, 128);
    if (tile == 11) return hipErrorInvalidValue;
  }
  if (tile == 2 || tile == 12) return launch_cfg<CfgMid, IN_DT, OUT_DT>(a, st);
  if (tile == 5) return launch_cfg<CfgSmallK4, IN_DT, OUT_DT>(a, st);
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
// 2 = 128x128, 3 = 256x256 (direct-to-LDS loads), 4 = 64x64 tiles with K cut into slices over workgroups,
// 5 = 64x64 tiles walked by four groups of waves.
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
  if (tile == 14) { a.c_blocked = 1; tile = 13; }
  switch (in_dt) {
    case DT_BF16: return launch_in<DT_BF16>(a, out_dt, tile, st);
    case DT_F16: return launch_in<DT_F16>(a, out_dt, tile, st);
    case DT_FP8: return launch_in<DT_FP8>(a, out_dt, tile, st);
  }
  return hipErrorInvalidValue;
}

// ---- K-sliced GEMM on a fixed scratch array -------------------------------------------------------
// For callers that cannot allocate device memory: the partial sums of the K slices live in an array that is part of
// the library's device image, one copy per GPU that loads it, held until the process ends. The array's name is a
// host-side stand-in; the address the kernels take comes from hipGetSymbolAddress, once per device.
static __device__ __align__(256) float scratch[STATIC_WS_BYTES / sizeof(float)];
static float* g_scratch_ptr[16] = {};

// rc: hipErrorInvalidValue with *too_big set when the slices need more than the array holds.
hipError_t launch_gemm_static_ws(GemmArgs a, int in_dt, int out_dt, hipStream_t st, bool* too_big, size_t* need_bytes) {
  *too_big = false;
  *need_bytes = 0;
  if (a.M <= 0 || a.N <= 0) return hipSuccess;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= 16) return hipErrorInvalidDevice;
  float* ptr = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if (!g_scratch_ptr[dev]) {
      void* sym = nullptr;
      e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));   // the current device's copy of the array
      if (e != hipSuccess) return e;
      g_scratch_ptr[dev] = static_cast<float*>(sym);
    }
    ptr = g_scratch_ptr[dev];
  }
  // The plan crl_gemm's tile 4 would make (its own workspace is larger than this one): same slices or refuse.
  GemmArgs plan = a;
  plan.splitk_ws = nullptr;
  int per = 0;
  const int ks = splitk_plan(plan, in_dt == DT_FP8 ? 1 : 2, true, &per);
  const size_t need = ks > 1 ? (size_t)ks * a.M * ((a.N + 7) / 8 * 8) * sizeof(float) : 0;
  *need_bytes = need;
  if (need > STATIC_WS_BYTES) { *too_big = true; return hipErrorInvalidValue; }
  a.splitk_ws = ptr;
  a.splitk_ws_bytes = (long)STATIC_WS_BYTES;
  return launch_gemm(a, in_dt, out_dt, 4, st);
}

}  // namespace crl