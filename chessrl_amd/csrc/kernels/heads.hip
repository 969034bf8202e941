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


template <int IN_DT>
__global__ void __launch_bounds__(256) policy_qk_kernel(const PolicyQKArgs a) {
  __shared__ float s_a[64 * 65];
  __shared__ float s_off[8][4];
  const int b = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lr = lane & 31, g = lane >> 5;
  const int it = wave & 1, jt = wave >> 1;
  const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + ((long)b * 64 + 32 * it + lr) * a.ldq + 8 * g;
  const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k) + ((long)b * 64 + 32 * jt + lr) * a.ldk + 8 * g;

  f32x16_t acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  const int steps = a.C / 16;
#pragma unroll 8
  for (int s = 0; s < steps; ++s) {
    const uint4 qv = *reinterpret_cast<const uint4*>(qp + 16 * s);
    const uint4 kv = *reinterpret_cast<const uint4*>(kp + 16 * s);
    if constexpr (IN_DT == DT_BF16)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kv), __builtin_bit_cast(bf16x8_t, qv), acc, 0, 0, 0);
    else
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, kv), __builtin_bit_cast(f16x8_t, qv), acc, 0, 0, 0);
  }
  // acc[r]: key j = 32jt + 8(r/4) + 4g + r%4, query i = 32it + lr.
  const int i = 32 * it + lr;
  if (a.dense) {
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      const int j = 32 * jt + 8 * rq + 4 * g;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = acc[4 * rq + e] * a.scale;
      const long off = (long)b * a.ldd + i * 64 + j;
      if (a.dense_dtype == DT_F32) {
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(a.dense) + off) = make_float4(v[0], v[1], v[2], v[3]);
      } else if (a.dense_dtype == DT_BF16) {
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(a.dense) + off) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
      } else {
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(a.dense) + off) =
            make_uint2((uint32_t)f32_to_f16_bits(v[0]) | ((uint32_t)f32_to_f16_bits(v[1]) << 16),
                       (uint32_t)f32_to_f16_bits(v[2]) | ((uint32_t)f32_to_f16_bits(v[3]) << 16));
      }
    }
  }
  if (!a.logits) return;  // uniform across the workgroup

#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int j = 32 * jt + 8 * (r >> 2) + 4 * g + (r & 3);
    s_a[i * 65 + j] = acc[r] * a.scale;
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
      for (int c = part; c < a.C; c += 8) {
        const float kv = (IN_DT == DT_BF16) ? bf16_bits_to_f32(krow[c]) : f16_bits_to_f32(krow[c]);
        sum = fmaf(kv, wrow[c], sum);
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
  if (a.C % 16 || a.ldq % 8 || a.ldk % 8 || (reinterpret_cast<uintptr_t>(a.q) & 15) || (reinterpret_cast<uintptr_t>(a.k) & 15))
    return hipErrorInvalidValue;
  if (a.dense && (a.ldd % 4)) return hipErrorInvalidValue;
  if (a.logits && (!a.gidx || !a.gpromo)) return hipErrorInvalidValue;
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
