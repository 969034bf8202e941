// Policy-head kernels.
//
//  * policy_qk: per position, A = Q·K^T / sqrt(d_model) over the 64 squares, the
//    attention-policy product of BT4.forward (new_paradigm/value.py:176-185). It either
//    writes the dense 4096 from-to logits (the reference then applies
//    Linear(4096->1929), value.py:187) or gathers them, together with promotion
//    offsets, into the 1858-move vocabulary (the BT4-class head).
//  * masked_softmax: logits + (1-mask)*(-999), divided by T, softmax; T == 0 selects
//    the arg-max (model_bis.py:382-392, new_paradigm/value.py:231-240).
//  * leela_to_rl: scatter of a 1858-entry row into the 1929-entry vocabulary with the
//    rank mirror for black rows (Leela/compare_policy.py:493-523).
#include "common.hpp"

namespace crl {


// One workgroup per position, four waves. Each wave takes a quarter of the channels and forms its partial 64x64 product
// from rows it alone reads (a row's 512 bytes of that quarter are four whole lines; with the channels shared and the
// output split over the waves instead, every row was fetched by two waves in 32-byte pieces: 2.4 TB/s); the partial
// tiles meet in LDS and are added in a fixed order, (w0 + w2) + (w1 + w3).
constexpr int PQK_STRIDE = 68;   // floats per row of a partial tile: 16 lanes' 16-byte stores cover 64 banks
template <int IN_DT>
__global__ void __launch_bounds__(256) policy_qk_kernel(const PolicyQKArgs a) {
  __shared__ __align__(16) float s_part[2][64 * PQK_STRIDE];
  __shared__ float s_off[8][4];
  float* const s_a = s_part[0];   // after the sum: the scaled 64x64 tile, row stride 65 (the gather's bank spread)
  const int b = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lr = lane & 31, g = lane >> 5;
  const int kq = a.C / 4;   // channels per wave (the launcher checks C % 64 == 0)
  const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + ((long)b * 64 + lr) * a.ldq + wave * kq + 8 * g;
  const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k) + ((long)b * 64 + lr) * a.ldk + wave * kq + 8 * g;
  const long q32 = 32 * a.ldq, k32 = 32 * a.ldk;

  f32x16_t acc[2][2];   // [jt][it]
#pragma unroll
  for (int jt = 0; jt < 2; ++jt)
#pragma unroll
    for (int it = 0; it < 2; ++it)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[jt][it][r] = 0.f;
  const int steps = kq / 16;
#pragma unroll 4
  for (int s = 0; s < steps; ++s) {
    uint4 qv[2], kv[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      qv[t] = *reinterpret_cast<const uint4*>(qp + t * q32 + 16 * s);
      kv[t] = *reinterpret_cast<const uint4*>(kp + t * k32 + 16 * s);
    }
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int it = 0; it < 2; ++it) {
        if constexpr (IN_DT == DT_BF16)
          acc[jt][it] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kv[jt]), __builtin_bit_cast(bf16x8_t, qv[it]), acc[jt][it], 0, 0, 0);
        else
          acc[jt][it] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, kv[jt]), __builtin_bit_cast(f16x8_t, qv[it]), acc[jt][it], 0, 0, 0);
      }
  }
  // acc[jt][it][r]: key j = 32jt + 8(r/4) + 4g + r%4, query i = 32it + lr.
  // Waves 0 and 1 lay their tiles down, waves 2 and 3 add theirs on top (same lane, same element).
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    if ((wave >> 1) == pass) {
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int it = 0; it < 2; ++it)
#pragma unroll
          for (int rq = 0; rq < 4; ++rq) {
            f32x4_t v4 = {acc[jt][it][4 * rq], acc[jt][it][4 * rq + 1], acc[jt][it][4 * rq + 2], acc[jt][it][4 * rq + 3]};
            f32x4_t* slot = reinterpret_cast<f32x4_t*>(&s_part[wave & 1][(32 * it + lr) * PQK_STRIDE + 32 * jt + 8 * rq + 4 * g]);
            if (pass == 1) v4 = *slot + v4;
            *slot = v4;
          }
    }
    __syncthreads();
  }
  // Thread t adds the two sums of row t / 4, columns [16 (t % 4), +16).
  float tot[16];
  {
    const int i = threadIdx.x >> 2, j0 = (threadIdx.x & 3) * 16;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const f32x4_t p0 = *reinterpret_cast<const f32x4_t*>(&s_part[0][i * PQK_STRIDE + j0 + 4 * c]);
      const f32x4_t p1 = *reinterpret_cast<const f32x4_t*>(&s_part[1][i * PQK_STRIDE + j0 + 4 * c]);
#pragma unroll
      for (int e = 0; e < 4; ++e) tot[4 * c + e] = (p0[e] + p1[e]) * a.scale;
    }
    if (a.dense) {
      const long off = (long)b * a.ldd + i * 64 + j0;
      if (a.dense_dtype == DT_F32) {
#pragma unroll
        for (int c = 0; c < 4; ++c)
          *reinterpret_cast<float4*>(reinterpret_cast<float*>(a.dense) + off + 4 * c) = make_float4(tot[4 * c], tot[4 * c + 1], tot[4 * c + 2], tot[4 * c + 3]);
      } else {
        uint32_t w[8];
#pragma unroll
        for (int e = 0; e < 8; ++e)
          w[e] = a.dense_dtype == DT_BF16 ? pack_bf16x2(tot[2 * e], tot[2 * e + 1])
                                          : ((uint32_t)f32_to_f16_bits(tot[2 * e]) | ((uint32_t)f32_to_f16_bits(tot[2 * e + 1]) << 16));
        uint4* dp = reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(a.dense) + off);
        dp[0] = make_uint4(w[0], w[1], w[2], w[3]);
        dp[1] = make_uint4(w[4], w[5], w[6], w[7]);
      }
    }
  }
  if (!a.logits) return;  // uniform across the workgroup

  __syncthreads();   // every thread has read its partials: their first tile becomes the summed one
  {
    const int i = threadIdx.x >> 2, j0 = (threadIdx.x & 3) * 16;
#pragma unroll
    for (int e = 0; e < 16; ++e) s_a[i * 65 + j0 + e] = tot[e];
  }
  // Promotion offsets from the keys of the promotion rank: tokens 0..7 when white is
  // to move, 56..63 (rank 1) when black is. 32 dot products, 8 threads each.
  const int white = a.white_to_move ? a.white_to_move[b] : 1;
  {
    const int dot = threadIdx.x >> 3, part = threadIdx.x & 7;
    const int file = dot >> 2, piece = dot & 3;
    const int tok = (white ? 0 : 56) + file;
    const uint16_t* krow = reinterpret_cast<const uint16_t*>(a.k) + ((long)b * 64 + tok) * a.ldk;
    const float* wrow = a.wpromo + (long)piece * a.C;
    float sum = 0.f;
    if (a.wpromo) {
      // (eight channels per thread and step: a 16-byte piece of the key row against two vectors of the weight row)
      for (int c = part * 8; c < a.C; c += 64) {
        const uint4 kraw = *reinterpret_cast<const uint4*>(krow + c);
        const float4 w0 = *reinterpret_cast<const float4*>(wrow + c), w1 = *reinterpret_cast<const float4*>(wrow + c + 4);
        const uint32_t kw[4] = {kraw.x, kraw.y, kraw.z, kraw.w};
        const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint16_t bits = (uint16_t)((e & 1) ? (kw[e >> 1] >> 16) : (kw[e >> 1] & 0xffff));
          sum = fmaf((IN_DT == DT_BF16) ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits), wv[e], sum);
        }
      }
    }
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    sum += __shfl_xor(sum, 4, 64);
    if (part == 0) s_off[file][piece] = sum;
  }
  __syncthreads();
  const int16_t* gi = a.gidx + (white ? a.nmoves : 0);
  for (int v = threadIdx.x; v < a.nmoves; v += 256) {
    const int ft = gi[v];
    float x = s_a[(ft >> 6) * 65 + (ft & 63)];
    const int pr = a.gpromo[v];
    if (pr >= 0) x += s_off[pr >> 2][pr & 3] + s_off[pr >> 2][3];
    a.logits[(long)b * a.ldl + v] = x;
  }
}

hipError_t launch_policy_qk(const PolicyQKArgs& a, hipStream_t st) {
  if (a.B <= 0) return hipSuccess;
  if (a.C % 64 || a.ldq % 8 || a.ldk % 8 || (reinterpret_cast<uintptr_t>(a.q) & 15) || (reinterpret_cast<uintptr_t>(a.k) & 15))
    return hipErrorInvalidValue;
  if (a.dense && ((a.ldd % 8) || (reinterpret_cast<uintptr_t>(a.dense) & 15))) return hipErrorInvalidValue;
  if (a.logits && (!a.gidx || !a.gpromo)) return hipErrorInvalidValue;
  if (a.wpromo && (reinterpret_cast<uintptr_t>(a.wpromo) & 15)) return hipErrorInvalidValue;
  if (a.in_dtype == DT_BF16) hipLaunchKernelGGL((policy_qk_kernel<DT_BF16>), dim3(a.B), dim3(256), 0, st, a);
  else if (a.in_dtype == DT_F16) hipLaunchKernelGGL((policy_qk_kernel<DT_F16>), dim3(a.B), dim3(256), 0, st, a);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

// ---- masked softmax ---------------------------------------------------------------------

__global__ void __launch_bounds__(256) masked_softmax_kernel(const SoftmaxArgs a) {
  __shared__ float s_red[4];
  __shared__ int s_idx[4];
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* lg = a.logits + (long)b * a.ldl;
  const uint8_t* mk = a.mask ? a.mask + (long)b * a.ldm : nullptr;
  const float inv_t = a.temperature > 0.f ? 1.0f / a.temperature : 1.0f;
  constexpr int PER = 8;  // covers V <= 2048
  float x[PER];
  float mx = -INFINITY;
  int mi = 0x7fffffff;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int v = e * 256 + tid;
    if (v < a.V) {
      float l = lg[v];
      if (mk) l += (1.0f - (float)mk[v]) * -999.0f;
      x[e] = l;
      if (l > mx) { mx = l; mi = v; }
    } else {
      x[e] = -INFINITY;
    }
  }
  // arg-max with the lowest index winning ties
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float om = __shfl_xor(mx, o, 64);
    const int oi = __shfl_xor(mi, o, 64);
    if (om > mx || (om == mx && oi < mi)) { mx = om; mi = oi; }
  }
  if (lane == 0) { s_red[wave] = mx; s_idx[wave] = mi; }
  __syncthreads();
  mx = s_red[0]; mi = s_idx[0];
#pragma unroll
  for (int w = 1; w < 4; ++w)
    if (s_red[w] > mx || (s_red[w] == mx && s_idx[w] < mi)) { mx = s_red[w]; mi = s_idx[w]; }
  if (a.argmax && tid == 0) a.argmax[b] = mi;
  if (!a.probs) return;
  float* pr = a.probs + (long)b * a.ldp;
  if (a.temperature <= 0.f) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int v = e * 256 + tid;
      if (v < a.V) pr[v] = (v == mi) ? 1.0f : 0.0f;
    }
    return;
  }
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int v = e * 256 + tid;
    if (v < a.V) { x[e] = expf((x[e] - mx) * inv_t); sum += x[e]; }
  }
  sum = wave_sum(sum);
  __syncthreads();
  if (lane == 0) s_red[wave] = sum;
  __syncthreads();
  sum = s_red[0] + s_red[1] + s_red[2] + s_red[3];
  const float inv = 1.0f / sum;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int v = e * 256 + tid;
    if (v < a.V) pr[v] = x[e] * inv;
  }
}

hipError_t launch_masked_softmax(const SoftmaxArgs& a, hipStream_t st) {
  if (a.B <= 0) return hipSuccess;
  if (a.V <= 0 || a.V > 2048) return hipErrorInvalidValue;
  hipLaunchKernelGGL(masked_softmax_kernel, dim3(a.B), dim3(256), 0, st, a);
  return hipGetLastError();
}

// ---- 1858 -> 1929 scatter ---------------------------------------------------------------------

__global__ void __launch_bounds__(256) leela_to_rl_kernel(const ScatterArgs a) {
  const int b = blockIdx.x;
  const int32_t* inv = a.white_to_move[b] ? a.inv_white : a.inv_black;
  for (int v = threadIdx.x; v < a.ndst; v += 256) {
    const int s = inv[v];
    a.dst[(long)b * a.ldd + v] = s >= 0 ? a.src[(long)b * a.lds + s] : 0.0f;
  }
}

hipError_t launch_leela_to_rl(const ScatterArgs& a, hipStream_t st) {
  if (a.B <= 0) return hipSuccess;
  hipLaunchKernelGGL(leela_to_rl_kernel, dim3(a.B), dim3(256), 0, st, a);
  return hipGetLastError();
}


// Side to move of each position: plane 12 of its first token (utils/fen_encoder.py:22).
// With the compact board form it is byte 0 of the position's four flag bytes.
__global__ void extract_stm_kernel(const float* planes, const uint8_t* flags, uint8_t* out, int B) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  out[b] = planes ? (planes[(long)b * 64 * 19 + 12] > 0.5f ? 1 : 0) : (flags[(long)b * 4] ? 1 : 0);
}
// ---- per-row log-softmax statistics ---------------------------------------------------------
// Serves the cross-entropy of GPT.forward(compute_loss=True) (model_bis.py:192-193) and the
// scoring terms of GRPO (grpo_refactored.py:337-342: log_softmax of the policy and the frozen
// reference model, the per-token KL and the log-probabilities of the tokens taken).
// One wave per row; the row (and the reference row) stays in registers, so each logit is read
// from memory once. V <= 64 * TS_VPL.
constexpr int TS_VPL = 32;

template <int WITH_REF>
__global__ void __launch_bounds__(256) token_score_kernel(const TokenScoreArgs a) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  const float* x = a.logits + (long)row * a.ldl;
  const float* y = WITH_REF ? a.ref + (long)row * a.ldr : nullptr;
  float xv[TS_VPL], yv[WITH_REF ? TS_VPL : 1];
  float mx = -INFINITY, my = -INFINITY;
#pragma unroll
  for (int i = 0; i < TS_VPL; ++i) {
    const int c = i * 64 + lane;
    xv[i] = c < a.V ? x[c] : -INFINITY;
    mx = fmaxf(mx, xv[i]);
    if constexpr (WITH_REF) {
      yv[i] = c < a.V ? y[c] : -INFINITY;
      my = fmaxf(my, yv[i]);
    }
  }
  mx = wave_max(mx);
  if constexpr (WITH_REF) my = wave_max(my);
  float sx = 0.f, sy = 0.f;
#pragma unroll
  for (int i = 0; i < TS_VPL; ++i) {
    sx += __expf(xv[i] - mx);
    if constexpr (WITH_REF) sy += __expf(yv[i] - my);
  }
  sx = wave_sum(sx);
  const float lse_x = mx + __logf(sx);
  float lse_y = 0.f;
  if constexpr (WITH_REF) {
    sy = wave_sum(sy);
    lse_y = my + __logf(sy);
    if (a.kl) {
      float k = 0.f;
#pragma unroll
      for (int i = 0; i < TS_VPL; ++i) {
        const int c = i * 64 + lane;
        if (c < a.V) {
          const float lp = xv[i] - lse_x;
          k += __expf(lp) * (lp - (yv[i] - lse_y));
        }
      }
      k = wave_sum(k);
      if (lane == 0) a.kl[row] = k;
    }
  }
  if (a.target && (a.logp || a.ref_logp)) {
    const long t = a.target[row];
    const bool ok = t != a.ignore_index && t >= 0 && t < a.V;
    if (lane == 0) {
      if (a.logp) a.logp[row] = ok ? x[t] - lse_x : 0.f;
      if (WITH_REF && a.ref_logp) a.ref_logp[row] = ok ? y[t] - lse_y : 0.f;
    }
  }
}

hipError_t launch_token_scores(const TokenScoreArgs& a, hipStream_t st) {
  if (a.rows <= 0) return hipSuccess;
  if (!a.logits || a.V <= 0 || a.V > 64 * TS_VPL) return hipErrorInvalidValue;
  if ((a.kl || a.ref_logp) && !a.ref) return hipErrorInvalidValue;
  const dim3 grid((a.rows + 3) / 4), block(256);
  if (a.ref) hipLaunchKernelGGL((token_score_kernel<1>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((token_score_kernel<0>), grid, block, 0, st, a);
  return hipGetLastError();
}

// One workgroup, fixed order: every thread sums a strided slice, then a tree over the workgroup.
__global__ void __launch_bounds__(256) masked_nll_mean_kernel(const float* logp, const int64_t* target, long ignore_index, int rows, float* out) {
  __shared__ float s_sum[256];
  __shared__ int s_cnt[256];
  float sum = 0.f;
  int cnt = 0;
  for (int r = threadIdx.x; r < rows; r += 256)
    if (target[r] != ignore_index) { sum -= logp[r]; ++cnt; }
  s_sum[threadIdx.x] = sum;
  s_cnt[threadIdx.x] = cnt;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) { s_sum[threadIdx.x] += s_sum[threadIdx.x + o]; s_cnt[threadIdx.x] += s_cnt[threadIdx.x + o]; }
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = s_cnt[0] > 0 ? s_sum[0] / (float)s_cnt[0] : 0.f;
}

hipError_t launch_masked_nll_mean(const float* logp, const int64_t* target, long ignore_index, int rows, float* out, hipStream_t st) {
  if (!logp || !target || !out || rows < 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(masked_nll_mean_kernel, dim3(1), dim3(256), 0, st, logp, target, ignore_index, rows, out);
  return hipGetLastError();
}

hipError_t launch_extract_stm(const float* planes, const uint8_t* flags, uint8_t* white_to_move, int B, hipStream_t st) {
  if (B <= 0) return hipSuccess;
  hipLaunchKernelGGL(extract_stm_kernel, dim3((B + 255) / 256), dim3(256), 0, st, planes, flags, white_to_move, B);
  return hipGetLastError();
}

// fp32 -> {f32, bf16, f16, e4m3(value*scale)} element conversion used when weights are packed.
__global__ void convert_kernel(const float* src, void* dst, long n, int dt, float scale) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float v = src[i];
  if (dt == DT_F32) reinterpret_cast<float*>(dst)[i] = v;
  else if (dt == DT_BF16) reinterpret_cast<uint16_t*>(dst)[i] = f32_to_bf16_bits(v);
  else if (dt == DT_F16) reinterpret_cast<uint16_t*>(dst)[i] = f32_to_f16_bits(v);
  else reinterpret_cast<uint8_t*>(dst)[i] = f32_to_fp8(v * scale);
}
hipError_t launch_convert(const float* src, void* dst, long n, int dt, float scale, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(convert_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, src, dst, n, dt, scale);
  return hipGetLastError();
}

__global__ void widen_kernel(const void* src, int dt, float* dst, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  dst[i] = dt == DT_F32 ? reinterpret_cast<const float*>(src)[i]
         : dt == DT_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(src)[i])
                         : f16_bits_to_f32(reinterpret_cast<const uint16_t*>(src)[i]);
}
hipError_t launch_widen(const void* src, int dt, float* dst, long n, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  if (dt != DT_F32 && dt != DT_BF16 && dt != DT_F16) return hipErrorInvalidValue;
  hipLaunchKernelGGL(widen_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, src, dt, dst, n);
  return hipGetLastError();
}

__global__ void fill_f32_kernel(float* p, float v, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
hipError_t launch_fill_f32(float* p, float v, long n, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p, v, n);
  return hipGetLastError();
}

}  // namespace crl
