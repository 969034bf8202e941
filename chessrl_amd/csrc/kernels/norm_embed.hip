// Row-wise LayerNorm and the board-token embedding.
//
// LayerNorm replaces F.layer_norm / nn.LayerNorm (eps 1e-5, affine) at
// model_bis.py:34, new_paradigm/value.py:36-37,134 and utils/fen_encoder.py:57; the
// residual sum it normalises is produced by the preceding GEMM's epilogue. It can
// also emit an e4m3 copy of its output (value * scale) so the next fp8 GEMM needs no
// separate quantise pass.
//
// The embedding kernel is FenEncoder.forward (utils/fen_encoder.py:61-67) and the
// identical stem of BT4.forward (new_paradigm/value.py:159-167): Linear(19->C), GELU,
// LayerNorm, x*exp(a)+b gating, plus the fixed sinusoid rows of model_bis.py:362-366
// when a table is supplied.
//
// One 64-lane wave owns one row; a lane keeps VPL vectors of 8 consecutive columns in
// registers, so a row is read once and the statistics are two wave reductions.
#include "common.hpp"

namespace crl {

template <int DT>
__device__ __forceinline__ void load8(const void* base, long off, float v[8]) {
  if constexpr (DT == DT_F32) {
    const float4* p = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + off);
    float4 a = p[0], b = p[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    uint4 u = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(base) + off);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (DT == DT_BF16) {
        v[2 * i] = bf16_bits_to_f32((uint16_t)(w[i] & 0xffff));
        v[2 * i + 1] = bf16_bits_to_f32((uint16_t)(w[i] >> 16));
      } else {
        v[2 * i] = f16_bits_to_f32((uint16_t)(w[i] & 0xffff));
        v[2 * i + 1] = f16_bits_to_f32((uint16_t)(w[i] >> 16));
      }
    }
  }
}

__device__ __forceinline__ void store8(void* base, long off, const float v[8], int dt) {
  if (dt == DT_F32) {
    float4* p = reinterpret_cast<float4*>(reinterpret_cast<float*>(base) + off);
    p[0] = make_float4(v[0], v[1], v[2], v[3]);
    p[1] = make_float4(v[4], v[5], v[6], v[7]);
  } else if (dt == DT_BF16) {
    uint4 u = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
    *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(base) + off) = u;
  } else {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_f16_bits(v[2 * i]) | ((uint32_t)f32_to_f16_bits(v[2 * i + 1]) << 16);
    *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(base) + off) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

__device__ __forceinline__ void store8_fp8(uint8_t* base, long off, const float v[8], float scale) {
  uint2 u = make_uint2(pack_fp8x4(v[0] * scale, v[1] * scale, v[2] * scale, v[3] * scale),
                       pack_fp8x4(v[4] * scale, v[5] * scale, v[6] * scale, v[7] * scale));
  *reinterpret_cast<uint2*>(base + off) = u;
}

// Normalise the VPL*8 values a lane holds (columns col0(i) = (i*64+lane)*8) and write them.
// rms: RMSNorm (mean taken as zero, no offset): y = x * rsqrt(mean(x^2) + eps) * gamma.
// FULL: C == VPL * 512, every lane holds VPL whole vectors (no column guards in the instruction stream).
template <int VPL, bool FULL = false>
__device__ __forceinline__ void ln_finish(float (&x)[VPL][8], int lane, int C, const float* gamma, const float* beta,
                                           float eps, float (&y)[VPL][8], float* stats = nullptr, bool rms = false) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    if (FULL || (i * 64 + lane) * 8 < C) {
#pragma unroll
      for (int e = 0; e < 8; ++e) s += x[i][e];
    }
  }
  // (1 / C by the hardware reciprocal, exact for the power-of-two widths and within one unit in the last place otherwise:
  // two IEEE divisions are 22 of a row's ~400 instructions)
  const float inv_c = fast_rcp((float)C);
  const float mean = rms ? 0.f : wave_sum(s) * inv_c;
  if (rms) beta = nullptr;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    if (FULL || (i * 64 + lane) * 8 < C) {
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float d = x[i][e] - mean; q += d * d; }
    }
  }
  const float rstd = rsqrtf(wave_sum(q) * inv_c + eps);
  if (stats && lane == 0) *reinterpret_cast<float2*>(stats) = make_float2(rstd, -mean * rstd);   // (x - mean) * rstd = x * s0 + s1
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = (i * 64 + lane) * 8;
    if (FULL || col < C) {
      float gv[8], bv[8];
      load8<DT_F32>(gamma, col, gv);
      if (beta) load8<DT_F32>(beta, col, bv);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[i][e] = (x[i][e] - mean) * rstd * gv[e] + (beta ? bv[e] : 0.f);
    }
  }
}

template <int IN_DT, int VPL, bool FULL = false>
__global__ void __launch_bounds__(256) layernorm_kernel(const LayerNormArgs a) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  float x[VPL][8], y[VPL][8];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = (i * 64 + lane) * 8;
    if (FULL || col < a.C) load8<IN_DT>(a.x, (long)row * a.ldx + col, x[i]);
  }
  ln_finish<VPL, FULL>(x, lane, a.C, a.gamma, a.beta, a.eps, y, a.stats ? a.stats + 2 * (long)row : nullptr, a.rms != 0);
  float am = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = (i * 64 + lane) * 8;
    if (FULL || col < a.C) {
      if (a.out) store8(a.out, (long)row * a.ldo + col, y[i], a.out_dtype);
      if (a.out_b) store8(a.out_b, (long)row * a.ldo + col, y[i], a.out_b_dtype);
      if (a.out_fp8) store8_fp8(a.out_fp8, (long)row * a.ldo + col, y[i], a.fp8_scale);
      if (a.amax) {
#pragma unroll
        for (int e = 0; e < 8; ++e) am = fmaxf(am, fabsf(y[i][e]));
      }
    }
  }
  if (a.amax) {
    am = wave_max(am);
    if (lane == 0) atomic_amax(a.amax, am);
  }
}

// The trunk's norm: bf16 rows of exactly 1024 elements, LayerNorm with offset, outputs bf16 and/or e4m3. Same arithmetic per
// row as layernorm_kernel (same order of additions, same roundings), but with everything about the call fixed at compile
// time and all of a wave's loads (RPW rows, then scale and offset, which RPW rows share) issued before the first
// reduction, so that a wave waits for memory once instead of three times.
template <bool OUT16, bool OUT8, int RPW>
__global__ void __launch_bounds__(256) layernorm_trunk_kernel(const LayerNormArgs a) {
  const int lane = threadIdx.x & 63;
  const long row0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW;
  if (row0 >= a.rows) return;
  float x[RPW][2][8], g[2][8], b[2][8];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    load8<DT_F32>(a.gamma, (i * 64 + lane) * 8, g[i]);
    load8<DT_F32>(a.beta, (i * 64 + lane) * 8, b[i]);
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      // (read once: with the non-temporal hint the row does not displace what the products around this launch keep in
      // the caches; measured on a 4096-position pass: this kernel -2.8 %, the pass -0.6 ms)
      typedef int i32x4_nt __attribute__((ext_vector_type(4)));
      const i32x4_nt raw = __builtin_nontemporal_load(reinterpret_cast<const i32x4_nt*>(reinterpret_cast<const uint16_t*>(a.x) + (row0 + r) * a.ldx + (i * 64 + lane) * 8));
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[r][i][2 * e] = bf16_bits_to_f32((uint16_t)((uint32_t)raw[e] & 0xffff));
        x[r][i][2 * e + 1] = bf16_bits_to_f32((uint16_t)((uint32_t)raw[e] >> 16));
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);   // (no use of a loaded value, and so no wait, moves up between the loads)
  const float inv_c = fast_rcp(1024.f);
  float am = 0.f;
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int e = 0; e < 8; ++e) s += x[r][i][e];
    }
    const float mean = wave_sum(s) * inv_c;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float d = x[r][i][e] - mean; q += d * d; }
    }
    const float rstd = rsqrtf(wave_sum(q) * inv_c + a.eps);
    if (a.stats && lane == 0) *reinterpret_cast<float2*>(a.stats + 2 * (row0 + r)) = make_float2(rstd, -mean * rstd);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      float y[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = (x[r][i][e] - mean) * rstd * g[i][e] + b[i][e];
      const long off = (row0 + r) * a.ldo + (i * 64 + lane) * 8;
      if constexpr (OUT16) store8(a.out, off, y, DT_BF16);
      if constexpr (OUT8) store8_fp8(a.out_fp8, off, y, a.fp8_scale);
      if (a.amax) {
#pragma unroll
        for (int e = 0; e < 8; ++e) am = fmaxf(am, fabsf(y[e]));
      }
    }
  }
  if (a.amax) {
    am = wave_max(am);
    if (lane == 0) atomic_amax(a.amax, am);
  }
}

template <int RPW>
static bool launch_ln_trunk(const LayerNormArgs& a, hipStream_t st) {
  const dim3 grid((a.rows / RPW + 3) / 4), block(256);
  if (a.out && a.out_fp8) hipLaunchKernelGGL((layernorm_trunk_kernel<true, true, RPW>), grid, block, 0, st, a);
  else if (a.out) hipLaunchKernelGGL((layernorm_trunk_kernel<true, false, RPW>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((layernorm_trunk_kernel<false, true, RPW>), grid, block, 0, st, a);
  return true;
}

// Rows longer than 2048 elements (the 8192-wide norm of the bias generator): the four waves of a workgroup share one
// row, 8 elements per thread and step of 2048, and meet through LDS for the two reductions (wave sums added in wave
// order). Chosen by the row length alone, so a row's result does not depend on how many rows the call has; with one
// row per position it also puts four times as many waves on a small batch as one wave per row would.
template <int IN_DT>
__global__ void __launch_bounds__(256) layernorm_wide_kernel(const LayerNormArgs a) {
  constexpr int VPT = 4;
  __shared__ float s_red[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long row = blockIdx.x;
  float x[VPT][8];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int col = (i * 256 + tid) * 8;
    if (col < a.C) {
      load8<IN_DT>(a.x, row * a.ldx + col, x[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) s += x[i][e];
    }
  }
  s = wave_sum(s);
  if (lane == 0) s_red[0][wave] = s;
  __syncthreads();
  const bool rms = a.rms != 0;
  const float mean = rms ? 0.f : (((s_red[0][0] + s_red[0][1]) + s_red[0][2]) + s_red[0][3]) / (float)a.C;
  const float* beta = rms ? nullptr : a.beta;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if ((i * 256 + tid) * 8 < a.C) {
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float d = x[i][e] - mean; q += d * d; }
    }
  }
  q = wave_sum(q);
  if (lane == 0) s_red[1][wave] = q;
  __syncthreads();
  const float rstd = rsqrtf((((s_red[1][0] + s_red[1][1]) + s_red[1][2]) + s_red[1][3]) / (float)a.C + a.eps);
  float am = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int col = (i * 256 + tid) * 8;
    if (col < a.C) {
      float gv[8], bv[8], y[8];
      load8<DT_F32>(a.gamma, col, gv);
      if (beta) load8<DT_F32>(beta, col, bv);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = (x[i][e] - mean) * rstd * gv[e] + (beta ? bv[e] : 0.f);
      if (a.out) store8(a.out, row * a.ldo + col, y, a.out_dtype);
      if (a.out_b) store8(a.out_b, row * a.ldo + col, y, a.out_b_dtype);
      if (a.out_fp8) store8_fp8(a.out_fp8, row * a.ldo + col, y, a.fp8_scale);
      if (a.amax) {
#pragma unroll
        for (int e = 0; e < 8; ++e) am = fmaxf(am, fabsf(y[e]));
      }
    }
  }
  if (a.amax) {
    am = wave_max(am);
    if (lane == 0) atomic_amax(a.amax, am);
  }
}

template <int IN_DT>
static hipError_t launch_ln_dt(const LayerNormArgs& a, hipStream_t st) {
  const dim3 grid((a.rows + 3) / 4), block(256);
  const int vecs = (a.C / 8 + 63) / 64;
  if constexpr (IN_DT == DT_BF16) {
    if (a.C == 1024 && !a.rms && a.beta && !a.out_b && (a.out || a.out_fp8) && (!a.out || a.out_dtype == DT_BF16)) {
      // (two rows per wave: 18 % faster than one at 262144 rows, and no slower than four; per-row arithmetic is the same)
      if (a.rows % 2 == 0) launch_ln_trunk<2>(a, st);
      else launch_ln_trunk<1>(a, st);
      return hipGetLastError();
    }
  }
  if (vecs <= 1) hipLaunchKernelGGL((layernorm_kernel<IN_DT, 1>), grid, block, 0, st, a);
  else if (a.C == 1024) hipLaunchKernelGGL((layernorm_kernel<IN_DT, 2, true>), grid, block, 0, st, a);   // (the trunk's width: no column guards)
  else if (vecs <= 2) hipLaunchKernelGGL((layernorm_kernel<IN_DT, 2>), grid, block, 0, st, a);
  else if (vecs <= 4) hipLaunchKernelGGL((layernorm_kernel<IN_DT, 4>), grid, block, 0, st, a);
  else if (vecs <= 16) hipLaunchKernelGGL((layernorm_wide_kernel<IN_DT>), dim3(a.rows), block, 0, st, a);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_layernorm(const LayerNormArgs& a, hipStream_t st) {
  if (a.rows <= 0) return hipSuccess;
  if (a.C % 8 || a.ldx % 8 || a.ldo % 8 || a.C > 8192) return hipErrorInvalidValue;
  if ((a.out && a.out_dtype == DT_FP8) || (a.out_b && a.out_b_dtype == DT_FP8)) return hipErrorInvalidValue;   // e4m3 goes through out_fp8
  if (a.stats && a.C > 2048) return hipErrorInvalidValue;   // the four-waves-per-row kernel does not write them
  switch (a.in_dtype) {
    case DT_F32: return launch_ln_dt<DT_F32>(a, st);
    case DT_BF16: return launch_ln_dt<DT_BF16>(a, st);
    case DT_F16: return launch_ln_dt<DT_F16>(a, st);
  }
  return hipErrorInvalidValue;
}

// ---- embedding ------------------------------------------------------------------------
template <int VPL>
__global__ void __launch_bounds__(256) embed_kernel(const EmbedArgs a) {
  const int lane = threadIdx.x & 63;
  const int tok = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tok >= a.tokens) return;
  const int sqr = tok & 63;

  // The 19 input features of this token (uniform across the wave).
  float f[19];
  if (a.planes) {
#pragma unroll
    for (int p = 0; p < 19; ++p) f[p] = a.planes[(long)tok * 19 + p];
  } else {
    const int b = tok >> 6;
    const int id = a.ids[tok];
    const uint8_t* fl = a.flags + b * 4;
#pragma unroll
    for (int p = 0; p < 12; ++p) f[p] = (id == p + 1) ? 1.f : 0.f;
    f[12] = fl[0] ? 1.f : 0.f;
    f[13] = (fl[2] == sqr) ? 1.f : 0.f;
    f[14] = (fl[1] & 1) ? 1.f : 0.f;
    f[15] = (fl[1] & 2) ? 1.f : 0.f;
    f[16] = (fl[1] & 4) ? 1.f : 0.f;
    f[17] = (fl[1] & 8) ? 1.f : 0.f;
    f[18] = fminf((float)fl[3] / 100.0f, 1.0f);
  }

  float x[VPL][8], y[VPL][8];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = (i * 64 + lane) * 8;
    if (col < a.C) {
      load8<DT_F32>(a.b1, col, x[i]);
#pragma unroll
      for (int p = 0; p < 19; ++p) {
        if (f[p] != 0.f) {  // uniform branch: most planes are zero for a given token
          float w[8];
          load8<DT_F32>(a.w1t, (long)p * a.C + col, w);
#pragma unroll
          for (int e = 0; e < 8; ++e) x[i][e] = fmaf(f[p], w[e], x[i][e]);
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) x[i][e] = apply_act(x[i][e], a.act);
    }
  }
  ln_finish<VPL>(x, lane, a.C, a.ln_g, a.ln_b, a.eps, y);
  const long orow = a.out_T > 64 ? (long)(tok >> 6) * a.out_T + sqr : (long)tok;
  float am = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int col = (i * 64 + lane) * 8;
    if (col < a.C) {
      float ga[8], gb[8];
      load8<DT_F32>(a.gate_a_exp, (long)sqr * a.C + col, ga);
      load8<DT_F32>(a.gate_b, (long)sqr * a.C + col, gb);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[i][e] = y[i][e] * ga[e] + gb[e];
      if (a.pe) {
        float pe[8];
        load8<DT_F32>(a.pe, (long)sqr * a.C + col, pe);
#pragma unroll
        for (int e = 0; e < 8; ++e) y[i][e] += pe[e];
      }
      store8(a.out, orow * a.C + col, y[i], a.out_dtype);
      if (a.out_b) store8(a.out_b, orow * a.C + col, y[i], a.out_b_dtype);
      if (a.out_fp8) store8_fp8(a.out_fp8, orow * a.C + col, y[i], a.fp8_scale);
      if (a.amax) {
#pragma unroll
        for (int e = 0; e < 8; ++e) am = fmaxf(am, fabsf(y[i][e]));
      }
    }
  }
  if (a.amax) {
    am = wave_max(am);
    if (lane == 0) atomic_amax(a.amax, am);
  }
}

// One workgroup per (position, move token).
__global__ void __launch_bounds__(256) token_embed_kernel(const TokenEmbedArgs a) {
  const int b = blockIdx.x / a.t, j = blockIdx.x - b * a.t;
  long id = a.idx[(long)b * a.t + j];
  id = id < 0 ? 0 : id >= a.V ? a.V - 1 : id;
  const float* w = a.wte + id * a.C;
  const float* pe = a.pe + (long)(64 + j) * a.C;
  const long row = (long)b * a.T + 64 + j;
  for (int c = threadIdx.x; c < a.C; c += 256) {
    const float v = w[c] + pe[c];
    if (a.out_dtype == DT_F32) reinterpret_cast<float*>(a.out)[row * a.C + c] = v;
    else if (a.out_dtype == DT_BF16) reinterpret_cast<uint16_t*>(a.out)[row * a.C + c] = f32_to_bf16_bits(v);
    else reinterpret_cast<uint16_t*>(a.out)[row * a.C + c] = f32_to_f16_bits(v);
  }
}

hipError_t launch_token_embed(const TokenEmbedArgs& a, hipStream_t st) {
  if (a.B <= 0 || a.t <= 0) return hipSuccess;
  if (!a.idx || !a.wte || !a.pe || !a.out || a.T != 64 + a.t || a.out_dtype == DT_FP8) return hipErrorInvalidValue;
  hipLaunchKernelGGL(token_embed_kernel, dim3(a.B * a.t), dim3(256), 0, st, a);
  return hipGetLastError();
}

hipError_t launch_embed(const EmbedArgs& a, hipStream_t st) {
  if (a.tokens <= 0) return hipSuccess;
  if (a.C % 8 || a.C > 2048) return hipErrorInvalidValue;
  const dim3 grid((a.tokens + 3) / 4), block(256);
  const int vecs = (a.C / 8 + 63) / 64;
  if (vecs <= 1) hipLaunchKernelGGL((embed_kernel<1>), grid, block, 0, st, a);
  else if (vecs <= 2) hipLaunchKernelGGL((embed_kernel<2>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((embed_kernel<4>), grid, block, 0, st, a);
  return hipGetLastError();
}

}  // namespace crl
