// Shared device helpers for the gfx950 kernels: element types, vector aliases,
// conversions, activations, 64-lane wave reductions and the kernel argument blocks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>

namespace crl {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));

// Element type codes used across the C ABI.
enum DType : int { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2, DT_FP8 = 3 };
enum Act : int { ACT_NONE = 0, ACT_GELU = 1, ACT_MISH = 2, ACT_SWISH = 3 };

__host__ __device__ inline int dtype_size(int dt) { return dt == DT_F32 ? 4 : dt == DT_FP8 ? 1 : 2; }

// ---- scalar conversions ------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
// Round-to-nearest-even through the gfx950 conversion instruction (v_cvt_pk_bf16_f32).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }

// OCP e4m3fn: 4 values -> 4 bytes with hardware saturating conversion (max 448).
__device__ __forceinline__ uint32_t pack_fp8x4(float a, float b, float c, float d) {
  a = fminf(fmaxf(a, -448.f), 448.f);
  b = fminf(fmaxf(b, -448.f), 448.f);
  c = fminf(fmaxf(c, -448.f), 448.f);
  d = fminf(fmaxf(d, -448.f), 448.f);
  int v = 0;
  v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, v, false);
  v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
  return (uint32_t)v;
}
__device__ __forceinline__ uint8_t f32_to_fp8(float a) {
  a = fminf(fmaxf(a, -448.f), 448.f);
  int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, a, 0, false);
  return (uint8_t)(v & 0xff);
}
__device__ __forceinline__ float fp8_to_f32(uint8_t b) { return __builtin_amdgcn_cvt_f32_fp8((int)b, 0); }

// ---- activations ---------------------------------------------------------------
// All three are straight-line code (no per-lane branch, hardware reciprocal instead of the IEEE division sequence):
// they run on every element of the GEMM epilogues, where the library forms (erff with its two divergent ranges,
// the early return of mish, precise division) cost 20-50 instructions and a branch per element.
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
// erf by Abramowitz & Stegun 7.1.26: |error| <= 1.5e-7 over the whole line.
__device__ __forceinline__ float erf_as(float x) {
  const float ax = fabsf(x);
  const float t = fast_rcp(fmaf(0.3275911f, ax, 1.0f));
  float p = fmaf(1.061405429f, t, -1.453152027f);
  p = fmaf(p, t, 1.421413741f);
  p = fmaf(p, t, -0.284496736f);
  p = fmaf(p, t, 0.254829592f);
  const float y = 1.0f - p * t * __expf(-ax * ax);
  return copysignf(y, x);
}
__device__ __forceinline__ float act_gelu(float x) { return 0.5f * x * (1.0f + erf_as(x * 0.70710678118654752f)); }
// mish(x) = x * tanh(softplus(x)); with n = e^x, tanh(log(1+n)) = (n^2+2n)/(n^2+2n+2). Past x = 20 the ratio is 1 in
// fp32, so the exponent is clamped there (n^2 would overflow from x = 44).
__device__ __forceinline__ float act_mish(float x) {
  const float n = __expf(fminf(x, 20.f));
  const float t = n * (n + 2.f);
  return x * (t * fast_rcp(t + 2.f));
}
__device__ __forceinline__ float act_swish(float x) { return x * fast_rcp(1.0f + __expf(-x)); }
__device__ __forceinline__ float apply_act(float x, int act) {
  switch (act) {
    case ACT_GELU: return act_gelu(x);
    case ACT_MISH: return act_mish(x);
    case ACT_SWISH: return act_swish(x);
    default: return x;
  }
}

// ---- wave reductions (64 lanes) ---------------------------------------------------
// An xor butterfly over lane distances 1, 2, 4, 8, 16, 32. The four short distances are data-parallel-primitive moves
// inside a row of 16 lanes (no trip through the LDS crossbar, which is what __shfl_xor compiles to: six dependent ones per
// reduction were most of a LayerNorm wave's latency). At distance 4 and 8 the partner is the mirrored lane of the half row
// or row: after the shorter steps every lane of a group of 4 or 8 holds the group's partial result, so the mirrored lane
// holds exactly what the xor partner holds.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_HALF_MIRROR = 0x141, DPP_MIRROR = 0x140;
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<DPP_XOR1>(v);
  v += dpp_move<DPP_XOR2>(v);
  v += dpp_move<DPP_HALF_MIRROR>(v);
  v += dpp_move<DPP_MIRROR>(v);
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<DPP_XOR1>(v));
  v = fmaxf(v, dpp_move<DPP_XOR2>(v));
  v = fmaxf(v, dpp_move<DPP_HALF_MIRROR>(v));
  v = fmaxf(v, dpp_move<DPP_MIRROR>(v));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

// amax is kept as the bit pattern of a non-negative float so integer max orders it.
__device__ __forceinline__ void atomic_amax(float* slot, float v) {
  atomicMax(reinterpret_cast<unsigned int*>(slot), __float_as_uint(v));
}

// ---- argument blocks ---------------------------------------------------------------
struct GemmArgs {
  const void* A;      // activations [M,K], row stride lda elements
  const void* W;      // weights [N,K] (nn.Linear layout), row stride ldw elements
  void* C;            // output [M,N], row stride ldc elements
  void* C2;           // optional second output for columns >= nsplit (written at column n-nsplit)
  const float* bias;  // [N] fp32 or null
  const void* res;    // optional residual [M,N], row stride ldr elements
  float* amax;        // optional: max |output| is accumulated here
  long lda, ldw, ldc, ldc2, ldr;
  int M, N, K;
  int nsplit;         // N if unused
  int act;            // Act
  int res_dtype;      // DType of res (bf16 or f32)
  float descale;      // multiplies the accumulator (1/(scale_a*scale_w) for fp8 inputs)
  float alpha;        // multiplies act(acc*descale+bias) before the residual is added
  float out_scale;    // multiplies the final value before an fp8 store
  int vec_ok;         // 1 if 4-wide stores/loads along N are aligned for C, C2 and res
  int res_rows;       // >0: the residual has this many rows and row m reads row m % res_rows
  int stream_out;     // 1: the output is far larger than the L2 caches: store it with the non-temporal hint
  int k_slices;       // >1: workgroup (tile, slice) covers slabs_per_slice 128-byte slabs of K and writes slice `slice` of C [k_slices, M, ldc]
  int slabs_per_slice;
  float* splitk_ws;   // workspace of the K-sliced path owned by the caller (else the library's per-stream one), splitk_ws_bytes long
  long splitk_ws_bytes;
  // Optional LayerNorm over the N columns of the result, written to ln_out (only where gemm_folds_layernorm says so).
  const float* ln_gamma; const float* ln_beta; void* ln_out; long ln_ldo; int ln_out_dtype; float ln_eps;
  int ln_rms;         // the folded norm is an RMSNorm (no mean subtraction, no offset)
  int k_parallel;     // 1: tile 0 may pick the K-sliced / K-grouped kernels, whose summation order over K differs from the tiled kernels'
  // Optional: the residual is LayerNorm(res) rather than res, normalised on the fly from the row statistics
  // res_stats [M,2] = (1/std, -mean/std) a LayerNorm launch left behind and that norm's gain and offset [N]
  // (256x256 tile with a 16-bit residual only; see gemm_takes_res_norm).
  const float* res_stats; const float* res_gamma; const float* res_beta;
  // 1: C (ldc == N) is written in contiguous blocks of 256 rows x 128 columns, block (m / 256, n / 128) at index
  // (m / 256) * (N / 128) + n / 128, instead of row-major (only where gemm_shortk_can says so).
  int c_blocked;
};

struct LayerNormArgs {
  const void* x;        // [rows, C]
  const float* gamma;   // [C]
  const float* beta;    // [C] or null
  void* out;            // optional [rows, C] in out_dtype
  uint8_t* out_fp8;     // optional [rows, C] e4m3, value*fp8_scale
  float* amax;          // optional
  long ldx, ldo;        // row strides in elements
  int rows, C;
  int in_dtype, out_dtype;
  float eps, fp8_scale;
  float* stats;         // optional [rows, 2]: 1/std and -mean/std of every row
  void* out_b;          // optional second copy [rows, C] in out_b_dtype (a 16-bit operand copy beside an fp32 residual copy)
  int out_b_dtype;
  int rms;              // 1: RMSNorm, y = x / sqrt(mean(x^2) + eps) * gamma (no mean subtraction, beta ignored)
};

struct EmbedArgs {
  const float* planes;  // [B*64, 19] or null when ids are given
  const uint8_t* ids;   // [B,64] piece codes 0..12 (token order), with flags
  const uint8_t* flags; // [B,4]
  const float* w1t;     // [19, C] (transposed linear1.weight)
  const float* b1;      // [C]
  const float* ln_g; const float* ln_b;   // [C]
  const float* gate_a_exp;  // [64, C] = exp(ma_gating.a)
  const float* gate_b;      // [64, C]
  const float* pe;          // optional [64, C] added after gating
  void* out;            // [B*64, C] in out_dtype
  uint8_t* out_fp8;     // optional
  void* out_b;          // optional second copy in out_b_dtype
  int out_b_dtype;
  float* amax;
  int tokens, C, out_dtype, act;
  float eps, fp8_scale;
  int out_T;            // rows per position in `out` (0 or 64: dense); token s of position b is written at row b*out_T + s
};

// Rows 64.. of a position that also carries move tokens: out[b*T + 64 + j] = wte[idx[b][j]] + pe[64 + j].
struct TokenEmbedArgs {
  const int64_t* idx;   // [B, t]
  const float* wte;     // [V, C]
  const float* pe;      // [>= T, C]
  void* out;            // [B*T, C] in out_dtype
  int B, t, T, C, V, out_dtype;
};

enum AttnMode : int { ATTN_PLAIN = 0, ATTN_CAUSAL = 1, ATTN_BIAS = 2, ATTN_RELSHIFT = 3 };

struct AttnArgs {
  const void* q; const void* k; const void* v;  // bf16 or f16, [B*64, ld*] with head h at column h*HS (q, k: h*qk_hstride if set)
  long ldq, ldk, ldv;
  int qk_hstride;       // elements between consecutive heads in q and in k; 0 = the head size. 2*HS with k = q + HS: [q_h | k_h] pairs,
                        // one whole 128-byte line per token and head at head size 32, which the kernel then reads with the non-temporal hint
  const void* bias;     // ATTN_BIAS: bf16 [B,H,4096] in the kernel's register order
  int bias_blocked;     // 1: the [B*H, 4096] bias matrix is stored in blocks of 256 rows x 128 columns (GemmArgs::c_blocked); B*H % 256 == 0
  const void* pos;      // ATTN_RELSHIFT: bf16 [64, H*HS] projected positional table
  const float* u_bias;  // ATTN_RELSHIFT: [H*HS]
  const float* v_bias;  // ATTN_RELSHIFT: [H*HS]
  void* out;            // [B*64, ldo] in the input element type, or fp8
  long ldo;
  float* amax;
  int B, H, mode, out_dtype;
  int T;                // tokens per position; 0 or 64 for the single-tile kernel, more only with ATTN_CAUSAL
  int in_dtype;         // DT_BF16 or DT_F16: element type of q, k, v, bias and pos
  float scale, out_scale;
};

struct PolicyQKArgs {
  const void* q; const void* k;   // bf16/f16 [B*64, ld], d_model contiguous
  long ldq, ldk;
  int in_dtype;                   // DT_BF16 or DT_F16
  int B, C;
  float scale;
  // dense mode
  void* dense; int dense_dtype; long ldd;   // [B, 4096], index = query*64 + key
  // gather mode
  float* logits; long ldl;                  // [B, 1858]
  const int16_t* gidx;                      // [2][1858] (black-to-move table first, then white): from_token*64+to_token
  const int8_t* gpromo;                     // [1858]: -1, or to_file*4 + piece (0 q, 1 r, 2 b)
  const float* wpromo;                      // [4, C] promotion offset weights (q, r, b, n)
  const uint8_t* white_to_move;             // [B]
  int nmoves;
};

struct SoftmaxArgs {
  const float* logits; long ldl;   // [B, V]
  const uint8_t* mask; long ldm;   // optional [B, V], 1 = legal
  float* probs; long ldp;          // optional [B, V]
  int32_t* argmax;                 // optional [B]
  int B, V;
  float temperature;               // 0 -> one-hot at the arg-max
};

// Per-row log-softmax statistics of a logits matrix.
struct TokenScoreArgs {
  const float* logits; long ldl;    // [rows, V]
  const float* ref; long ldr;       // optional second logits matrix [rows, V]
  const int64_t* target;            // optional [rows]
  float* logp;                      // optional [rows]: log_softmax(logits)[target] (0 where target is ignore_index or out of range)
  float* ref_logp;                  // optional [rows]: log_softmax(ref)[target]
  float* kl;                        // optional [rows]: sum_v softmax(logits)*(log_softmax(logits)-log_softmax(ref))
  int rows, V;
  long ignore_index;
};

// One sampling step of sequence generation.
struct SampleArgs {
  const float* logits; long ldl;     // [B, V]
  int64_t* seq; long ld_seq;         // [B, >= k+1]: token k is written, token k-2 is read by the rules
  int64_t* tok_out;                  // [B]: the same token, dense, for the next embedding
  int32_t* num_zeros;                // [B] end_variation counters (rules only)
  float* step_out; long ld_out;      // optional [B, V]: probabilities, or the raw logits when out_logits
  int B, V, k, step, rules, out_logits;
  long end_think, end_tok, end_variation;
  float temperature;
  uint64_t seed;
  const int* dyn_k;                  // optional device counter: k and step are read from it (graph replays), step_out advances with it
};

struct ScatterArgs {
  const float* src; long lds;       // [B, 1858]
  float* dst; long ldd;             // [B, 1929], fully written (zeros where no source)
  const int32_t* inv_white;         // [1929]: source index for a white row, or -1
  const int32_t* inv_black;         // [1929]: source index for a black row, or -1
  const uint8_t* white_to_move;     // [B]
  int B, nsrc, ndst;
};

// ---- launchers (one per kernel family) -------------------------------------------------
// in_dt: element type of A and W; out_dt: element type of C/C2; tile: 0 auto, 1 = 64x64,
// 2 = 128x128, 3 = 256x256 workgroup tile, 4 = 64x64 tiles with K cut into slices, 5 = 64x64 tiles whose K slabs four
// groups of waves take in turn. Tiles 1-3 add up K in the same order, so with tile 0 a row's result does not depend on
// how many other rows the call has; 4 and 5 are picked by tile 0 only when a.k_parallel is set (few tiles, where they
// are faster).
hipError_t launch_gemm(GemmArgs a, int in_dt, int out_dt, int tile, hipStream_t st);
// True when launch_gemm (tile 0) would take the K-sliced path for these arguments, whose second pass can apply the
// LayerNorm that follows the GEMM (GemmArgs::ln_*); launch_gemm rejects ln_out otherwise.
bool gemm_folds_layernorm(const GemmArgs& a, int in_dt);
// Whether the product can be written in the blocked layout of GemmArgs::c_blocked (gemm_shortk.hip has the one kernel that does).
bool gemm_shortk_can(const GemmArgs& a, int in_dt, int out_dt);
// crl_gemm's tile 4 with the slices' partial sums in a fixed array of the library's device image (no allocation).
constexpr size_t STATIC_WS_BYTES = 8u << 20;
hipError_t launch_gemm_static_ws(GemmArgs a, int in_dt, int out_dt, hipStream_t st, bool* too_big, size_t* need_bytes);
// Frees the device memory the GEMM launchers keep outside any model (per-stream K-slice workspaces, the zeros block).
void release_gemm_globals();
hipError_t launch_layernorm(const LayerNormArgs& a, hipStream_t st);
hipError_t launch_embed(const EmbedArgs& a, hipStream_t st);
hipError_t launch_token_embed(const TokenEmbedArgs& a, hipStream_t st);
hipError_t launch_token_scores(const TokenScoreArgs& a, hipStream_t st);
// mean of -logp over rows whose target is not ignore_index, in a fixed summation order; *out = 0 if there is none.
hipError_t launch_masked_nll_mean(const float* logp, const int64_t* target, long ignore_index, int rows, float* out, hipStream_t st);
hipError_t launch_attention(const AttnArgs& a, int head_dim, hipStream_t st);
hipError_t launch_policy_qk(const PolicyQKArgs& a, hipStream_t st);
hipError_t launch_masked_softmax(const SoftmaxArgs& a, hipStream_t st);
hipError_t launch_leela_to_rl(const ScatterArgs& a, hipStream_t st);
hipError_t launch_extract_stm(const float* planes, const uint8_t* flags, uint8_t* white_to_move, int B, hipStream_t st);
hipError_t launch_fill_f32(float* p, float v, long n, hipStream_t st);
hipError_t launch_convert(const float* src, void* dst, long n, int dt, float scale, hipStream_t st);
// {f32, bf16, f16} -> f32
hipError_t launch_widen(const void* src, int dt, float* dst, long n, hipStream_t st);
hipError_t launch_kv_store(const void* qkv, void* cache, int B, int T, int Tmax, int C, hipStream_t st);
// dyn_k (optional, device): the kernels take the token index k from it instead of from their arguments, so one captured
// graph serves every step: position = 64 + k, keys = 65 + k.
hipError_t launch_decode_embed(const int64_t* tok, const float* wte, const float* pe, int pos, const int* dyn_k, void* out, int B, int C, int V,
                               int out_dtype, hipStream_t st);
hipError_t launch_decode_attention(const void* q, long ldq, const void* cache, int Tmax, int C, int n, const int* dyn_k, void* out, long ldo,
                                   int B, int H, int head_dim, int in_dtype, float scale, hipStream_t st);
// staging [B, 2C] -> row (pos or 64 + *dyn_k) of every sequence's [Tmax, 2C] cache
hipError_t launch_kv_append(const void* staging, void* cache, int B, int Tmax, int C, int pos, const int* dyn_k, hipStream_t st);
hipError_t launch_add_int(int* p, int v, hipStream_t st);
hipError_t launch_sample(const SampleArgs& a, hipStream_t st);
// Back-to-back MFMAs from registers on every CU: sustained TFLOP/s and the clock it ran at.
hipError_t run_mfma_probe(int dtype, int random_bits, int iters, double* tflops, double* ghz, hipStream_t st);
hipError_t run_cu_split_probe(int gemm_cus, int tile, int rows, int iters, double* out8);
// Slot of (query i, key j) inside a 4096-element attention bias tile.
int attn_bias_slot_host(int i, int j);

}  // namespace crl
