// Incremental decoding for the GPT model: the kernels that let one new token per sequence be
// processed against cached keys and values instead of re-running the whole prefix, plus the
// on-device sampling step. Replaces the per-step full recomputation of
// GPT.generate_sequence / generate_sequence_raw (model_bis.py:213-263, 266-311).
#include "common.hpp"

namespace crl {

// ---- K|V of a freshly computed prefix into the cache ------------------------------------------
// qkv [B*T, 3C] (q|k|v per row) -> cache [B, Tmax, 2C] (k|v per row), 16-bit elements, 16 bytes per thread.
__global__ void __launch_bounds__(256) kv_store_kernel(const uint16_t* qkv, uint16_t* cache, int B, int T, int Tmax, int C) {
  const int chunks = 2 * C / 8;
  const long n = (long)B * T * chunks;
  for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const long row = i / chunks;
    const int c = (int)(i - row * chunks);
    const int b = (int)(row / T), s = (int)(row - (long)b * T);
    const uint4 v = *reinterpret_cast<const uint4*>(qkv + row * 3 * C + C + 8 * c);
    *reinterpret_cast<uint4*>(cache + ((long)b * Tmax + s) * 2 * C + 8 * c) = v;
  }
}

hipError_t launch_kv_store(const void* qkv, void* cache, int B, int T, int Tmax, int C, hipStream_t st) {
  if (B <= 0 || T <= 0) return hipSuccess;
  if (C % 8 || T > Tmax) return hipErrorInvalidValue;
  const long n = (long)B * T * (2 * C / 8);
  const int grid = (int)std::min<long>((n + 255) / 256, 8192);
  hipLaunchKernelGGL(kv_store_kernel, dim3(grid), dim3(256), 0, st, reinterpret_cast<const uint16_t*>(qkv), reinterpret_cast<uint16_t*>(cache), B, T, Tmax, C);
  return hipGetLastError();
}

// staging [B, 2C] (k|v of the newest token) -> its row of every sequence's cache
__global__ void __launch_bounds__(256) kv_append_kernel(const uint16_t* staging, uint16_t* cache, int B, int Tmax, int C, int pos, const int* dyn_k) {
  const int row = dyn_k ? 64 + dyn_k[0] : pos;
  const int chunks = 2 * C / 8;
  const int n = B * chunks;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const int b = i / chunks, c = i - b * chunks;
    *reinterpret_cast<uint4*>(cache + ((long)b * Tmax + row) * 2 * C + 8 * c) = *reinterpret_cast<const uint4*>(staging + (long)b * 2 * C + 8 * c);
  }
}

hipError_t launch_kv_append(const void* staging, void* cache, int B, int Tmax, int C, int pos, const int* dyn_k, hipStream_t st) {
  if (B <= 0) return hipSuccess;
  if (C % 8 || (!dyn_k && (pos < 0 || pos >= Tmax))) return hipErrorInvalidValue;
  const int n = B * (2 * C / 8);
  hipLaunchKernelGGL(kv_append_kernel, dim3(std::min((n + 255) / 256, 1024)), dim3(256), 0, st, reinterpret_cast<const uint16_t*>(staging),
                     reinterpret_cast<uint16_t*>(cache), B, Tmax, C, pos, dyn_k);
  return hipGetLastError();
}

__global__ void add_int_kernel(int* p, int v) { p[0] += v; }
hipError_t launch_add_int(int* p, int v, hipStream_t st) {
  hipLaunchKernelGGL(add_int_kernel, dim3(1), dim3(1), 0, st, p, v);
  return hipGetLastError();
}

// ---- embedding of the newest token -------------------------------------------------------------
// out[b] = wte[tok[b]] + pe[pos] (model_bis.py:224, 233-235 for the last position only).
__global__ void __launch_bounds__(256) decode_embed_kernel(const int64_t* tok, const float* wte, const float* pe, int pos, const int* dyn_k, void* out,
                                                           int C, int V, int out_dtype) {
  const int b = blockIdx.x;
  const float* pe_row = pe + (long)(dyn_k ? 64 + dyn_k[0] : pos) * C;
  long id = tok[b];
  id = id < 0 ? 0 : id >= V ? V - 1 : id;
  for (int c = threadIdx.x; c < C; c += 256) {
    const float v = wte[id * C + c] + pe_row[c];
    const long o = (long)b * C + c;
    if (out_dtype == DT_F32) reinterpret_cast<float*>(out)[o] = v;
    else if (out_dtype == DT_BF16) reinterpret_cast<uint16_t*>(out)[o] = f32_to_bf16_bits(v);
    else reinterpret_cast<uint16_t*>(out)[o] = f32_to_f16_bits(v);
  }
}

hipError_t launch_decode_embed(const int64_t* tok, const float* wte, const float* pe, int pos, const int* dyn_k, void* out, int B, int C, int V,
                               int out_dtype, hipStream_t st) {
  if (B <= 0) return hipSuccess;
  if (!tok || !wte || !pe || !out || out_dtype == DT_FP8) return hipErrorInvalidValue;
  hipLaunchKernelGGL(decode_embed_kernel, dim3(B), dim3(256), 0, st, tok, wte, pe, pos, dyn_k, out, C, V, out_dtype);
  return hipGetLastError();
}

// ---- one query against the cache -------------------------------------------------------------------
// One workgroup of four waves per (sequence, head). A key or value row of the head (HS elements) is read by HS/8
// neighbouring lanes, 16 bytes each, so a wave instruction covers 64/(HS/8) whole rows; the waves take such row groups
// in turn. Scores go to LDS, every wave derives the same max and sum from them, each wave accumulates p*V over its own
// rows, and the four partial outputs are added in wave order.
constexpr int DEC_TMAX = 1024;

template <int HS, int IN_DT>
__global__ void __launch_bounds__(256) decode_attention_kernel(const uint16_t* q, long ldq, const uint16_t* cache, int Tmax, int C, int n_arg,
                                                               const int* dyn_k, uint16_t* out, long ldo, int B, int H, float scale) {
  constexpr int LPK = HS / 8, KPI = 64 / LPK;    // lanes per key row, key rows per wave instruction
  __shared__ float s_p[DEC_TMAX];
  __shared__ float s_acc[4][HS];
  const int n = dyn_k ? 65 + dyn_k[0] : n_arg;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int sub = lane % LPK, kin = lane / LPK;
  const int unit = blockIdx.x;
  const int b = unit / H, h = unit - b * H;
  auto unpack = [](const uint4 u, float (&f)[8]) {
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint16_t x = (uint16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffff));
      f[e] = IN_DT == DT_BF16 ? bf16_bits_to_f32(x) : f16_bits_to_f32(x);
    }
  };
  float qv[8];
  unpack(*reinterpret_cast<const uint4*>(q + (long)b * ldq + h * HS + sub * 8), qv);
  const uint16_t* kbase = cache + (long)b * Tmax * 2 * C + h * HS + sub * 8;

#pragma unroll 4
  for (int j0 = wave * KPI; j0 < n; j0 += 4 * KPI) {
    const int j = j0 + kin;
    float s = 0.f;
    if (j < n) {
      float kv[8];
      unpack(*reinterpret_cast<const uint4*>(kbase + (long)j * 2 * C), kv);
#pragma unroll
      for (int e = 0; e < 8; ++e) s = fmaf(qv[e], kv[e], s);
    }
#pragma unroll
    for (int o = 1; o < LPK; o <<= 1) s += __shfl_xor(s, o, 64);
    if (sub == 0 && j < n) s_p[j] = s * scale;
  }
  __syncthreads();
  float mx = -INFINITY;
  for (int j = lane; j < n; j += 64) mx = fmaxf(mx, s_p[j]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = lane; j < n; j += 64) sum += __expf(s_p[j] - mx);
  sum = wave_sum(sum);

  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  const uint16_t* vbase = kbase + C;
#pragma unroll 4
  for (int j0 = wave * KPI; j0 < n; j0 += 4 * KPI) {
    const int j = j0 + kin;
    if (j < n) {
      const float pj = __expf(s_p[j] - mx);
      float vv[8];
      unpack(*reinterpret_cast<const uint4*>(vbase + (long)j * 2 * C), vv);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = fmaf(pj, vv[e], acc[e]);
    }
  }
#pragma unroll
  for (int o = LPK; o < 64; o <<= 1)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += __shfl_xor(acc[e], o, 64);
  if (kin == 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) s_acc[wave][sub * 8 + e] = acc[e];
  }
  __syncthreads();
  if (threadIdx.x < HS) {
    const int d = threadIdx.x;
    const float v = (((s_acc[0][d] + s_acc[1][d]) + s_acc[2][d]) + s_acc[3][d]) / sum;
    out[(long)b * ldo + h * HS + d] = IN_DT == DT_BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
  }
}

hipError_t launch_decode_attention(const void* q, long ldq, const void* cache, int Tmax, int C, int n, const int* dyn_k, void* out, long ldo,
                                   int B, int H, int head_dim, int in_dtype, float scale, hipStream_t st) {
  if (B <= 0) return hipSuccess;
  if (Tmax > DEC_TMAX || C % 8 || ldq % 8 || (reinterpret_cast<uintptr_t>(q) & 15) || (reinterpret_cast<uintptr_t>(cache) & 15) || (in_dtype != DT_BF16 && in_dtype != DT_F16)) return hipErrorInvalidValue;
  if (!dyn_k && (n < 1 || n > Tmax)) return hipErrorInvalidValue;
  const dim3 grid(B * H), block(256);
  const uint16_t* qp = reinterpret_cast<const uint16_t*>(q);
  const uint16_t* cp = reinterpret_cast<const uint16_t*>(cache);
  uint16_t* op = reinterpret_cast<uint16_t*>(out);
#define DEC_LAUNCH(HS, DT) hipLaunchKernelGGL((decode_attention_kernel<HS, DT>), grid, block, 0, st, qp, ldq, cp, Tmax, C, n, dyn_k, op, ldo, B, H, scale)
  if (head_dim == 32 && in_dtype == DT_BF16) DEC_LAUNCH(32, DT_BF16);
  else if (head_dim == 32) DEC_LAUNCH(32, DT_F16);
  else if (head_dim == 64 && in_dtype == DT_BF16) DEC_LAUNCH(64, DT_BF16);
  else if (head_dim == 64) DEC_LAUNCH(64, DT_F16);
  else return hipErrorInvalidValue;
#undef DEC_LAUNCH
  return hipGetLastError();
}

// ---- sampling ------------------------------------------------------------------------------------------
// One wave per sequence: softmax(logits/T) and one draw by inverse CDF (arg-max for T == 0), then the
// forced tokens of generate_sequence (model_bis.py:252-259) when rules != 0:
//   five end_variation tokens so far -> </thinking>; the token two places after </thinking> -> end.
// Lane l owns the contiguous classes [l*CH, l*CH+CH), so the CDF is a lane-level scan plus a short walk.
constexpr int SAMPLE_CH = 32;

__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t a, uint64_t b) {
  uint64_t z = seed + 0x9E3779B97F4A7C15ull * (a * 0x100000001B3ull + b + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

__global__ void __launch_bounds__(256) sample_kernel(const SampleArgs a) {
  const int lane = threadIdx.x & 63;
  const int b = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= a.B) return;
  const int k = a.dyn_k ? a.dyn_k[0] : a.k;
  const int step = a.dyn_k ? k : a.step;
  const float* x = a.logits + (long)b * a.ldl;
  const int ch = (a.V + 63) / 64;
  const float invT = a.temperature > 0.f ? 1.0f / a.temperature : 1.0f;
  float v[SAMPLE_CH];
  float mx = -INFINITY;
  int amax_i = 0x7fffffff;
#pragma unroll
  for (int i = 0; i < SAMPLE_CH; ++i) {
    const int c = lane * ch + i;
    v[i] = (i < ch && c < a.V) ? x[c] * invT : -INFINITY;
    if (v[i] > mx) { mx = v[i]; amax_i = c; }
  }
  // arg-max with the lowest index among equals
  float wmx = mx;
  int wi = amax_i;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float om = __shfl_xor(wmx, o, 64);
    const int oi = __shfl_xor(wi, o, 64);
    if (om > wmx || (om == wmx && oi < wi)) { wmx = om; wi = oi; }
  }
  float lsum = 0.f;
#pragma unroll
  for (int i = 0; i < SAMPLE_CH; ++i) {
    v[i] = __expf(v[i] - wmx);   // exp(-inf) = 0 for the padding
    lsum += v[i];
  }
  // inclusive scan of the lane sums
  float incl = lsum;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float t = __shfl_up(incl, o, 64);
    if (lane >= o) incl += t;
  }
  const float total = __shfl(incl, 63, 64);
  long tok = wi;
  if (a.temperature > 0.f) {
    const float target = uniform01(a.seed, (uint64_t)b, (uint64_t)step) * total;
    const float excl = incl - lsum;
    // the first lane whose inclusive sum exceeds the target holds the draw
    const bool mine = target < incl && target >= excl;
    int pick = -1;
    if (mine) {
      float run = excl;
      pick = lane * ch;
#pragma unroll
      for (int i = 0; i < SAMPLE_CH; ++i) {
        if (i < ch && lane * ch + i < a.V) {
          if (v[i] > 0.f) pick = lane * ch + i;    // last class with mass at or before the crossing
          run += v[i];
          if (run > target) break;
        }
      }
    }
    // rounding can leave no lane (target == total): fall back to the arg-max
    int found = pick;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) found = max(found, __shfl_xor(found, o, 64));
    if (found >= 0) tok = found;
  }
  if (a.step_out) {
    float* o = a.step_out + (long)b * a.ld_out + (a.dyn_k ? (long)(k - 1) * a.V : 0);
    const float inv = 1.0f / total;
#pragma unroll
    for (int i = 0; i < SAMPLE_CH; ++i) {
      const int c = lane * ch + i;
      if (i < ch && c < a.V) o[c] = a.out_logits ? x[c] : v[i] * inv;
    }
  }
  if (lane == 0) {
    if (a.rules) {
      int nz = a.num_zeros[b];
      if (nz == 5) { tok = a.end_think; nz = 6; }
      if (k >= 2 && a.seq[(long)b * a.ld_seq + k - 2] == a.end_think) tok = a.end_tok;
      nz += (tok == a.end_variation) ? 1 : 0;
      a.num_zeros[b] = nz;
    }
    a.seq[(long)b * a.ld_seq + k] = tok;
    a.tok_out[b] = tok;
  }
}

hipError_t launch_sample(const SampleArgs& a, hipStream_t st) {
  if (a.B <= 0) return hipSuccess;
  if (!a.logits || !a.seq || !a.tok_out || a.V <= 0 || a.V > 64 * SAMPLE_CH || (a.rules && !a.num_zeros)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_kernel, dim3((a.B + 3) / 4), dim3(256), 0, st, a);
  return hipGetLastError();
}

}  // namespace crl
