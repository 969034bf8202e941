// Fused 64-token multi-head attention: one 64-lane wave per (position, head).
//
// Replaces F.scaled_dot_product_attention(q,k,v,is_causal=True) of model_bis.py:71 and
// the score/softmax/context chain of RelativeMultiHeadAttention2.forward
// (new_paradigm/attn.py:507-521), including the pad-and-reshape relative shift of
// new_paradigm/attn.py:525-533. A third mode adds a generated per-head 64x64 bias
// before the softmax (the BT4-class configuration).
//
// The wave computes the TRANSPOSED score tile S^T[j][i] = K[j]·Q[i] with 32x32x16
// MFMAs whose operands are 16-byte row segments read straight from global memory
// (both Q and K are head-dim contiguous). In the accumulator layout a lane then owns
// one query i and 32 of its 64 keys j, so the softmax over keys is a reduction over
// the lane's own registers plus one exchange with lane^32. The probabilities are
// re-used in place as the column operand of the second product O^T = V^T · P^T; only V
// needs a transpose, which goes through a wave-private LDS patch.
#include "common.hpp"

namespace crl {

constexpr int VT_STRIDE = 68;   // bf16 elements per V^T row (64 keys + 4 padding: rows 8 apart land 16 banks apart, so the transposing
                                // 8-byte writes and the fragment reads of a wave touch every bank twice, the minimum; with 72 it was eight and four times)
constexpr int SP_STRIDE = 65;   // floats per row of the positional score patch

// Storage order of a 64x64 bias tile so that each lane reads its accumulator
// registers as 16-byte vectors: element (query i, key j) lives at
//   ((((i/32)*2 + j/32)*2 + rh)*64 + lane)*8 + e
// with lane = (i%32) + 32*g, j%32 = 8*(2*rh + e/4) + 4*g + e%4.
__host__ __device__ inline int attn_bias_slot(int i, int j) {
  const int it = i >> 5, jt = j >> 5, jj = j & 31;
  const int q4 = jj >> 3, g = (jj >> 2) & 1, e0 = jj & 3;
  const int rh = q4 >> 1, e = ((q4 & 1) << 2) | e0;
  const int lane = (i & 31) + 32 * g;
  return ((((it * 2 + jt) * 2 + rh) * 64 + lane) << 3) + e;
}

// The two 16-bit element types the kernel runs in.
template <int DT>
struct Half16;
template <>
struct Half16<DT_BF16> {
  typedef bf16x8_t vec;
  typedef __bf16 elem;
  static __device__ __forceinline__ f32x16_t mfma(vec a, vec b, f32x16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ float to_f32(uint16_t h) { return bf16_bits_to_f32(h); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
};
template <>
struct Half16<DT_F16> {
  typedef f16x8_t vec;
  typedef _Float16 elem;
  static __device__ __forceinline__ f32x16_t mfma(vec a, vec b, f32x16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ float to_f32(uint16_t h) { return f16_bits_to_f32(h); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return (uint32_t)f32_to_f16_bits(lo) | ((uint32_t)f32_to_f16_bits(hi) << 16); }
};

template <typename H>
__device__ __forceinline__ typename H::vec add_bias_h(typename H::vec q, const float* bias8) {
  typename H::vec r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (typename H::elem)((float)q[e] + bias8[e]);
  return r;
}

// Waves per workgroup: the relative-shift mode needs a 16.6 KB score patch per wave,
// so it runs two waves per workgroup to stay inside 64 KB of static LDS. With a generated bias a workgroup takes eight
// heads of a position (eight waves): per token row it then reads 512 contiguous bytes of each of q, k and v, its bias is
// 2 KB pieces of the blocked layout and its e4m3 output rows are two whole lines (measured 9.07 -> 8.53 ms per
// 4096-position forward against four waves; sixteen waves, one workgroup per CU, 9.71 ms).
template <int MODE>
struct AttnWaves { static constexpr int N = MODE == ATTN_RELSHIFT ? 2 : MODE == ATTN_BIAS ? 8 : 4; };

// Waves per SIMD the register allocation is held to (0: the compiler's own choice). The kernel is a chain of load,
// compute and store phases, so resident waves are what hides its memory latency: at head size 32 with a generated
// bias it fits 4 waves in 122 registers without spilling (152 and 3 waves left alone; measured 10.8 -> 9.6 ms per
// 4096-position forward; 5 waves spill and are slower). The other instances spill at that bound and keep theirs.
// 16 bytes that the kernel reads once: loaded with the non-temporal hint so that they do not displace what other kernels
// will want from the caches.
__device__ __forceinline__ uint4 attn_load_once(const void* p) {
  typedef int i32x4_nt __attribute__((ext_vector_type(4)));
  const i32x4_nt v = __builtin_nontemporal_load(reinterpret_cast<const i32x4_nt*>(p));
  return make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
}

template <int HS, int MODE>
struct AttnMinWaves { static constexpr int N = (HS == 32 && MODE == ATTN_BIAS) ? 4 : 0; };

// OUT_FP8: write e4m3 (value*out_scale) instead of the input element type.
// COOP: the workgroup's outputs leave through an LDS tile as whole row segments (see s_out below; the launcher says when).
template <int HS, int MODE, int OUT_FP8, int IN_DT, int COOP = 0>
__global__ void __launch_bounds__(64 * AttnWaves<MODE>::N, (AttnMinWaves<HS, MODE>::N)) attention_kernel(const AttnArgs a) {
  typedef Half16<IN_DT> H16;
  typedef typename H16::vec hvec;
  constexpr int KS = HS / 16;   // k-steps of the score product
  constexpr int DT_TILES = HS / 32;
  constexpr int NW = AttnWaves<MODE>::N;
  __shared__ __align__(16) uint16_t s_vt[NW][HS * VT_STRIDE];
  __shared__ float s_sp[MODE == ATTN_RELSHIFT ? NW : 1][MODE == ATTN_RELSHIFT ? 64 * SP_STRIDE : 1];
  // Output tile of the workgroup's NW heads (head size 32): 64 rows of NW * HS elements, 16 bytes of padding
  // per row. A wave's own output is 64 row pieces of 32 (e4m3) or 64 bytes, which it would have to store 16 bytes per
  // lane and row, a quarter or an eighth of a line at a time; gathered here, the workgroup stores whole lines (measured
  // on 4096 positions x 32 heads in e4m3: the stores were 9 % of the kernel's bytes and 21 % of its time).
  static_assert(!COOP || (HS == 32 && (NW == 4 || NW == 8 || NW == 16)), "the output tile is laid out for head size 32");
  constexpr int OSZ = OUT_FP8 ? 1 : 2;
  constexpr int OROW = NW * HS * OSZ, OSTRIDE = OROW + 16;
  __shared__ __align__(16) uint8_t s_out[COOP ? 64 * OSTRIDE : 16];

  // A wave that starts gets its loads out ahead of its neighbours' arithmetic: raised priority until the score product
  // begins (which also keeps every load above that point: 8.49 -> 8.31 ms per 4096-position forward).
  if constexpr (MODE == ATTN_BIAS) __builtin_amdgcn_s_setprio(3);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lr = lane & 31, g = lane >> 5;
  // (workgroup indices go round the eight XCDs: renumbered so that each XCD walks a contiguous range of units)
  int bid = blockIdx.x;
  {
    const int per = gridDim.x >> 3;
    if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
  }
  const int unit = bid * NW + wave;
  if (unit >= a.B * a.H) return;
  const int b = unit / a.H, h = unit - b * a.H;
  constexpr bool coop = COOP != 0;

  const int qk_hst = a.qk_hstride ? a.qk_hstride : HS;
  const bool qk_once = a.qk_hstride != 0;   // q and k of a head share lines with nobody else
  const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + (long)b * 64 * a.ldq + h * qk_hst;
  const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k) + (long)b * 64 * a.ldk + h * qk_hst;
  const uint16_t* vp = reinterpret_cast<const uint16_t*>(a.v) + (long)b * 64 * a.ldv + h * HS;

  // ---- V -> V^T in LDS ------------------------------------------------------------
  uint16_t* vt = s_vt[wave];
  // VPAIR: the two waves of a pair of neighbouring heads (a token's V rows of the two are one whole 128-byte line) take
  // half the tokens each, for both heads: every line is read by one wave, once, with the non-temporal hint, and lands
  // transposed in the patch of the head it belongs to; the workgroup meets at a barrier before the second product.
  constexpr bool VPAIR = COOP != 0 && MODE == ATTN_BIAS && HS == 32 && NW % 2 == 0;
  if constexpr (VPAIR) {
    const int half = wave & 1;
    const uint16_t* vp2 = vp - half * HS;
    const int dc8 = lane & 7, jq8 = lane >> 3;
    uint4 rows[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) rows[t] = attn_load_once(vp2 + (long)(32 * half + 4 * jq8 + t) * a.ldv + 8 * dc8);
    uint16_t* vt2 = s_vt[(wave & ~1) + (dc8 >> 2)];
    const int dc = dc8 & 3, jq = 8 * half + jq8;
    const uint32_t* w0 = reinterpret_cast<const uint32_t*>(&rows[0]);
    const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&rows[1]);
    const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&rows[2]);
    const uint32_t* w3 = reinterpret_cast<const uint32_t*>(&rows[3]);
#pragma unroll
    for (int e2 = 0; e2 < 4; ++e2) {
      uint2 lo = make_uint2((w0[e2] & 0xffffu) | (w1[e2] << 16), (w2[e2] & 0xffffu) | (w3[e2] << 16));
      uint2 hi = make_uint2((w0[e2] >> 16) | (w1[e2] & 0xffff0000u), (w2[e2] >> 16) | (w3[e2] & 0xffff0000u));
      *reinterpret_cast<uint2*>(vt2 + (8 * dc + 2 * e2) * VT_STRIDE + 4 * jq) = lo;
      *reinterpret_cast<uint2*>(vt2 + (8 * dc + 2 * e2 + 1) * VT_STRIDE + 4 * jq) = hi;
    }
  } else {
    constexpr int DC = HS / 8;            // 16-byte chunks per V row
    constexpr int PASSES = (16 * DC) / 64;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int id = p * 64 + lane;
      const int jq = id / DC, dc = id - jq * DC;
      uint4 rows[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) rows[t] = *reinterpret_cast<const uint4*>(vp + (long)(4 * jq + t) * a.ldv + 8 * dc);
      const uint32_t* w0 = reinterpret_cast<const uint32_t*>(&rows[0]);
      const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&rows[1]);
      const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&rows[2]);
      const uint32_t* w3 = reinterpret_cast<const uint32_t*>(&rows[3]);
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2) {
        // d = 8dc + 2e2 (low halves) and d+1 (high halves)
        uint2 lo = make_uint2((w0[e2] & 0xffffu) | (w1[e2] << 16), (w2[e2] & 0xffffu) | (w3[e2] << 16));
        uint2 hi = make_uint2((w0[e2] >> 16) | (w1[e2] & 0xffff0000u), (w2[e2] >> 16) | (w3[e2] & 0xffff0000u));
        *reinterpret_cast<uint2*>(vt + (8 * dc + 2 * e2) * VT_STRIDE + 4 * jq) = lo;
        *reinterpret_cast<uint2*>(vt + (8 * dc + 2 * e2 + 1) * VT_STRIDE + 4 * jq) = hi;
      }
    }
  }

  // ---- scores -----------------------------------------------------------------------
  hvec qf[2][KS], kf[2][KS];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const uint16_t* qa = qp + (long)(32 * t + lr) * a.ldq + 16 * ks + 8 * g;
      const uint16_t* ka = kp + (long)(32 * t + lr) * a.ldk + 16 * ks + 8 * g;
      if (qk_once) {
        qf[t][ks] = __builtin_bit_cast(hvec, attn_load_once(qa));
        kf[t][ks] = __builtin_bit_cast(hvec, attn_load_once(ka));
      } else {
        qf[t][ks] = *reinterpret_cast<const hvec*>(qa);
        kf[t][ks] = *reinterpret_cast<const hvec*>(ka);
      }
    }

  // The bias tile (8 KB per wave), requested behind V, q and k: loads return in the order of their issue, which is now
  // the order of their use, and all twenty are out before the first of them is waited for.
  uint4 braw[2][2][2];
  if constexpr (MODE == ATTN_BIAS) {
    // Element k = 512 L + 8 lane + e of the unit's 4096 (L = (it, jt, rh)): row-major, or in blocks of 256 units x 128
    // elements (the layout the bias generator's GEMM writes fastest), where a load of 1 KB is four pieces of 256 bytes.
    const uint16_t* bp = reinterpret_cast<const uint16_t*>(a.bias);
    long lstride = 512;
    if (a.bias_blocked) {
      bp += (long)(unit >> 8) * (256 * 4096) + ((long)(lane >> 4) * 256 + (unit & 255)) * 128 + ((lane & 15) << 3);
      lstride = 4 * 256 * 128;
    } else {
      bp += (long)unit * 4096 + (lane << 3);
    }
#pragma unroll
    for (int it = 0; it < 2; ++it)
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int rh = 0; rh < 2; ++rh)
          braw[it][jt][rh] = attn_load_once(bp + ((it * 2 + jt) * 2 + rh) * lstride);
  }

  if constexpr (MODE == ATTN_BIAS) __builtin_amdgcn_s_setprio(0);
  f32x16_t s[2][2];  // [jt][it]
#pragma unroll
  for (int jt = 0; jt < 2; ++jt)
#pragma unroll
    for (int it = 0; it < 2; ++it)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[jt][it][r] = 0.f;

  if constexpr (MODE == ATTN_RELSHIFT) {
    // content = (q+u)·k, position = (q+v)·p, both with the bias folded into the query.
    const uint16_t* pp = reinterpret_cast<const uint16_t*>(a.pos) + h * HS;
    const long ldp = (long)a.H * HS;
    f32x16_t sp[2][2];
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int it = 0; it < 2; ++it)
#pragma unroll
        for (int r = 0; r < 16; ++r) sp[jt][it][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      float ub[8], vb[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        ub[e] = a.u_bias[h * HS + 16 * ks + 8 * g + e];
        vb[e] = a.v_bias[h * HS + 16 * ks + 8 * g + e];
      }
      hvec pf[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) pf[t] = *reinterpret_cast<const hvec*>(pp + (long)(32 * t + lr) * ldp + 16 * ks + 8 * g);
#pragma unroll
      for (int it = 0; it < 2; ++it) {
        const hvec qu = add_bias_h<H16>(qf[it][ks], ub);
        const hvec qv = add_bias_h<H16>(qf[it][ks], vb);
#pragma unroll
        for (int jt = 0; jt < 2; ++jt) {
          s[jt][it] = H16::mfma(kf[jt][ks], qu, s[jt][it]);
          sp[jt][it] = H16::mfma(pf[jt], qv, sp[jt][it]);
        }
      }
    }
    // Shifted read-back (new_paradigm/attn.py:525-533): with T=64,
    //   out[i][j] = P[i][63-i+j] (j<=i), 0 (j==i+1), P[i+1][j-i-2] (j>i+1).
    float* spm = s_sp[wave];
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int it = 0; it < 2; ++it)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = 32 * jt + 8 * (r >> 2) + 4 * g + (r & 3);
          spm[(32 * it + lr) * SP_STRIDE + m] = sp[jt][it][r];
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int it = 0; it < 2; ++it)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = 32 * jt + 8 * (r >> 2) + 4 * g + (r & 3);
          const int i = 32 * it + lr;
          float pv;
          if (j <= i) pv = spm[i * SP_STRIDE + (63 - i + j)];
          else if (j == i + 1) pv = 0.f;
          else pv = spm[(i + 1) * SP_STRIDE + (j - i - 2)];
          s[jt][it][r] = (s[jt][it][r] + pv) * a.scale;
        }
  } else {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int it = 0; it < 2; ++it)
          s[jt][it] = H16::mfma(kf[jt][ks], qf[it][ks], s[jt][it]);

    if constexpr (MODE == ATTN_BIAS) {
#pragma unroll
      for (int it = 0; it < 2; ++it)
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
          for (int rh = 0; rh < 2; ++rh) {
            const uint4 u = braw[it][jt][rh];
            const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float bv = H16::to_f32((uint16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffff)));
              s[jt][it][8 * rh + e] = s[jt][it][8 * rh + e] * a.scale + bv;
            }
          }
    } else {
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int it = 0; it < 2; ++it)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float x = s[jt][it][r] * a.scale;
            if constexpr (MODE == ATTN_CAUSAL) {
              const int j = 32 * jt + 8 * (r >> 2) + 4 * g + (r & 3);
              const int i = 32 * it + lr;
              if (j > i) x = -INFINITY;
            }
            s[jt][it][r] = x;
          }
    }
  }

  // ---- softmax over keys (registers + lane^32) ------------------------------------------
  float inv_l[2];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    float mx = -INFINITY;
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[jt][it][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    float sum = 0.f;
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = __expf(s[jt][it][r] - mx);
        s[jt][it][r] = p;
        sum += p;
      }
    sum += __shfl_xor(sum, 32, 64);
    inv_l[it] = 1.0f / sum;
  }

  // ---- O^T = V^T · P^T ------------------------------------------------------------------
  if constexpr (VPAIR) {
    __syncthreads();   // (the other wave of the pair wrote half of this head's V^T)
  } else {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  f32x16_t o[DT_TILES][2];
#pragma unroll
  for (int dt = 0; dt < DT_TILES; ++dt)
#pragma unroll
    for (int it = 0; it < 2; ++it)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][it][r] = 0.f;

#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    const int jt = kb >> 1, kh = kb & 1;
    hvec pf[2];
#pragma unroll
    for (int it = 0; it < 2; ++it)
#pragma unroll
      for (int e = 0; e < 8; ++e) pf[it][e] = (typename H16::elem)s[jt][it][8 * kh + e];
#pragma unroll
    for (int dt = 0; dt < DT_TILES; ++dt) {
      const uint16_t* vrow = vt + (32 * dt + lr) * VT_STRIDE + 16 * kb + 4 * g;
      const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
      const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 8);
      const uint4 packed = make_uint4(lo.x, lo.y, hi.x, hi.y);
      const hvec vf = __builtin_bit_cast(hvec, packed);
#pragma unroll
      for (int it = 0; it < 2; ++it) o[dt][it] = H16::mfma(vf, pf[it], o[dt][it]);
    }
  }

  // ---- normalise and store ----------------------------------------------------------------
  float am = 0.f;
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const long row = (long)b * 64 + 32 * it + lr;
#pragma unroll
    for (int dt = 0; dt < DT_TILES; ++dt)
#pragma unroll
      for (int rp = 0; rp < 2; ++rp) {
        // A lane holds dims 8rq + 4g .. +3 of its row for rq = 0..3; the lane 32 away holds the other four of each
        // group of eight. The two swap one half per pair of groups, so each stores 8 consecutive dims of the row
        // (8 bytes of e4m3 or 16 bytes of 16-bit elements) and a row receives 16 or 32 contiguous bytes per instruction.
        uint32_t pk[2][2];   // [rq - 2rp][word]: e4m3 uses word 0 only
#pragma unroll
        for (int q2 = 0; q2 < 2; ++q2) {
          const int rq = 2 * rp + q2;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = o[dt][it][4 * rq + e] * inv_l[it];
            am = fmaxf(am, fabsf(v[e]));
          }
          if constexpr (OUT_FP8) {
            pk[q2][0] = pack_fp8x4(v[0] * a.out_scale, v[1] * a.out_scale, v[2] * a.out_scale, v[3] * a.out_scale);
            pk[q2][1] = 0;
          } else {
            pk[q2][0] = H16::pack2(v[0], v[1]);
            pk[q2][1] = H16::pack2(v[2], v[3]);
          }
        }
        // g = 0 keeps group 2rp and receives the partner's half of it; g = 1 keeps group 2rp+1.
        const int keep = g, give = 1 - g;
        const uint32_t r0 = __shfl_xor(pk[give][0], 32, 64);
        const int d = 32 * dt + 16 * rp + 8 * g;
        const long off = row * a.ldo + h * HS + d;
        if constexpr (OUT_FP8) {
          const uint2 w = g ? make_uint2(r0, pk[keep][0]) : make_uint2(pk[keep][0], r0);
          if constexpr (coop) *reinterpret_cast<uint2*>(s_out + (32 * it + lr) * OSTRIDE + (wave * HS + d) * OSZ) = w;
          else *reinterpret_cast<uint2*>(reinterpret_cast<uint8_t*>(a.out) + off) = w;
        } else {
          const uint32_t r1 = __shfl_xor(pk[give][1], 32, 64);
          const uint4 w = g ? make_uint4(r0, r1, pk[keep][0], pk[keep][1]) : make_uint4(pk[keep][0], pk[keep][1], r0, r1);
          if constexpr (coop) *reinterpret_cast<uint4*>(s_out + (32 * it + lr) * OSTRIDE + (wave * HS + d) * OSZ) = w;
          else *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(a.out) + off) = w;
        }
      }
  }
  if constexpr (COOP) {
    {
      __syncthreads();
      // 16-byte chunks of the tile, row by row: a wave-instruction stores 8 (e4m3) or 4 (16-bit) whole row segments.
      constexpr int CPR = OROW / 16;   // chunks per row
      char* const ob = reinterpret_cast<char*>(a.out) + ((long)b * 64 * a.ldo + (h - wave) * HS) * OSZ;
      const long ldo_b = a.ldo * OSZ;
#pragma unroll
      for (int i = 0; i < 64 * CPR / (64 * NW); ++i) {
        const int id = i * (64 * NW) + threadIdx.x;
        const int row = id / CPR, c = id % CPR;
        const uint4 w = *reinterpret_cast<const uint4*>(s_out + row * OSTRIDE + c * 16);
        *reinterpret_cast<uint4*>(ob + row * ldo_b + c * 16) = w;
      }
    }
  }
  if (a.amax) {
    am = wave_max(am);
    if (lane == 0) atomic_amax(a.amax, am);
  }
}

// Causal attention over T > 64 tokens per position (the board tokens followed by move tokens,
// model_bis.py:171-199 with F.scaled_dot_product_attention(is_causal=True) at :71). One wave per
// (position, head, block of 64 queries) walks the key blocks 0..own block with the running
// maximum and sum of a streaming softmax. In the transposed layout a lane owns one query in the
// score tile and in the output tile alike, so the rescale of the running output is one
// multiply per register with the lane's own factor.
template <int HS, int OUT_FP8, int IN_DT>
__global__ void __launch_bounds__(256) causal_long_kernel(const AttnArgs a) {
  typedef Half16<IN_DT> H16;
  typedef typename H16::vec hvec;
  constexpr int KS = HS / 16;
  constexpr int DT_TILES = HS / 32;
  __shared__ __align__(16) uint16_t s_vt[4][HS * VT_STRIDE];

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lr = lane & 31, g = lane >> 5;
  const int T = a.T, nqb = (T + 63) >> 6;
  const int unit = blockIdx.x * 4 + wave;
  if (unit >= a.B * a.H * nqb) return;
  // Longest units (last query block) first: they walk the most key blocks.
  const int qb = nqb - 1 - unit / (a.B * a.H);
  const int bh = unit % (a.B * a.H);
  const int b = bh / a.H, h = bh - b * a.H;
  const long row0 = (long)b * T;

  const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + row0 * a.ldq + h * HS;
  const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k) + row0 * a.ldk + h * HS;
  const uint16_t* vp = reinterpret_cast<const uint16_t*>(a.v) + row0 * a.ldv + h * HS;
  uint16_t* vt = s_vt[wave];
  auto clampT = [&](int t) { return t < T ? t : T - 1; };   // rows past the end re-read the last token

  hvec qf[2][KS];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[t][ks] = *reinterpret_cast<const hvec*>(qp + (long)clampT(64 * qb + 32 * t + lr) * a.ldq + 16 * ks + 8 * g);

  float run_m[2] = {-INFINITY, -INFINITY}, run_l[2] = {0.f, 0.f};
  f32x16_t o[DT_TILES][2];
#pragma unroll
  for (int dt = 0; dt < DT_TILES; ++dt)
#pragma unroll
    for (int it = 0; it < 2; ++it)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][it][r] = 0.f;

  for (int kb = 0; kb <= qb; ++kb) {
    // ---- V block -> V^T in LDS (the previous block's reads are complete: same wave, in order)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    {
      constexpr int DC = HS / 8;
      constexpr int PASSES = (16 * DC) / 64;
#pragma unroll
      for (int p = 0; p < PASSES; ++p) {
        const int id = p * 64 + lane;
        const int jq = id / DC, dc = id - jq * DC;
        uint4 rows[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) rows[t] = *reinterpret_cast<const uint4*>(vp + (long)clampT(64 * kb + 4 * jq + t) * a.ldv + 8 * dc);
        const uint32_t* w0 = reinterpret_cast<const uint32_t*>(&rows[0]);
        const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&rows[1]);
        const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&rows[2]);
        const uint32_t* w3 = reinterpret_cast<const uint32_t*>(&rows[3]);
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          uint2 lo = make_uint2((w0[e2] & 0xffffu) | (w1[e2] << 16), (w2[e2] & 0xffffu) | (w3[e2] << 16));
          uint2 hi = make_uint2((w0[e2] >> 16) | (w1[e2] & 0xffff0000u), (w2[e2] >> 16) | (w3[e2] & 0xffff0000u));
          *reinterpret_cast<uint2*>(vt + (8 * dc + 2 * e2) * VT_STRIDE + 4 * jq) = lo;
          *reinterpret_cast<uint2*>(vt + (8 * dc + 2 * e2 + 1) * VT_STRIDE + 4 * jq) = hi;
        }
      }
    }
    // ---- scores of this key block
    hvec kf[2][KS];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        kf[t][ks] = *reinterpret_cast<const hvec*>(kp + (long)clampT(64 * kb + 32 * t + lr) * a.ldk + 16 * ks + 8 * g);
    f32x16_t s[2][2];
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int it = 0; it < 2; ++it) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[jt][it][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s[jt][it] = H16::mfma(kf[jt][ks], qf[it][ks], s[jt][it]);
      }
    const bool edge = kb == qb;   // only the diagonal block needs the causal test; keys past T sit in it too
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int i = 64 * qb + 32 * it + lr;
      float mx = run_m[it];
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = 64 * kb + 32 * jt + 8 * (r >> 2) + 4 * g + (r & 3);
          float x = s[jt][it][r] * a.scale;
          if (edge && (j > i || j >= T)) x = -INFINITY;
          s[jt][it][r] = x;
          mx = fmaxf(mx, x);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      // Key 0 is visible to every query, so mx is finite from the first block on.
      const float alpha = __expf(run_m[it] - mx);
      float sum = 0.f;
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = __expf(s[jt][it][r] - mx);
          s[jt][it][r] = p;
          sum += p;
        }
      sum += __shfl_xor(sum, 32, 64);
      run_l[it] = run_l[it] * alpha + sum;
      run_m[it] = mx;
#pragma unroll
      for (int dt = 0; dt < DT_TILES; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][it][r] *= alpha;
    }
    // ---- O^T += V^T · P^T
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int k4 = 0; k4 < 4; ++k4) {
      const int jt = k4 >> 1, kh = k4 & 1;
      hvec pf[2];
#pragma unroll
      for (int it = 0; it < 2; ++it)
#pragma unroll
        for (int e = 0; e < 8; ++e) pf[it][e] = (typename H16::elem)s[jt][it][8 * kh + e];
#pragma unroll
      for (int dt = 0; dt < DT_TILES; ++dt) {
        const uint16_t* vrow = vt + (32 * dt + lr) * VT_STRIDE + 16 * k4 + 4 * g;
        const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
        const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 8);
        const uint4 packed = make_uint4(lo.x, lo.y, hi.x, hi.y);
        const hvec vf = __builtin_bit_cast(hvec, packed);
#pragma unroll
        for (int it = 0; it < 2; ++it) o[dt][it] = H16::mfma(vf, pf[it], o[dt][it]);
      }
    }
  }

  float am = 0.f;
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int i = 64 * qb + 32 * it + lr;
    if (i >= T) continue;
    const float inv_l = 1.0f / run_l[it];
    const long row = row0 + i;
#pragma unroll
    for (int dt = 0; dt < DT_TILES; ++dt)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int d = 32 * dt + 8 * rq + 4 * g;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = o[dt][it][4 * rq + e] * inv_l;
          am = fmaxf(am, fabsf(v[e]));
        }
        const long off = row * a.ldo + h * HS + d;
        if constexpr (OUT_FP8) {
          *reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(a.out) + off) =
              pack_fp8x4(v[0] * a.out_scale, v[1] * a.out_scale, v[2] * a.out_scale, v[3] * a.out_scale);
        } else {
          *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(a.out) + off) = make_uint2(H16::pack2(v[0], v[1]), H16::pack2(v[2], v[3]));
        }
      }
  }
  if (a.amax) {
    am = wave_max(am);
    if (lane == 0) atomic_amax(a.amax, am);
  }
}

template <int HS, int IN_DT>
static hipError_t launch_causal_long_dt(const AttnArgs& a, hipStream_t st) {
  const long units = (long)a.B * a.H * ((a.T + 63) / 64);
  const dim3 grid((unsigned)((units + 3) / 4)), block(256);
  if (a.out_dtype == DT_FP8) hipLaunchKernelGGL((causal_long_kernel<HS, 1, IN_DT>), grid, block, 0, st, a);
  else if (a.out_dtype == IN_DT) hipLaunchKernelGGL((causal_long_kernel<HS, 0, IN_DT>), grid, block, 0, st, a);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}
template <int HS>
static hipError_t launch_causal_long(const AttnArgs& a, hipStream_t st) {
  if (a.in_dtype == DT_F16) return launch_causal_long_dt<HS, DT_F16>(a, st);
  if (a.in_dtype == DT_BF16) return launch_causal_long_dt<HS, DT_BF16>(a, st);
  return hipErrorInvalidValue;
}

template <int HS, int MODE, int IN_DT>
static hipError_t launch_attn_dt(const AttnArgs& a, hipStream_t st) {
  constexpr int NW = AttnWaves<MODE>::N;
  const dim3 grid((a.B * a.H + NW - 1) / NW), block(64 * NW);
  if constexpr (HS == 32 && (NW == 4 || NW == 8 || NW == 16)) {
    // Whole workgroups only: H a multiple of 4 puts four heads of one position in every workgroup and leaves none partly
    // filled; 16-byte stores need rows and base aligned to that.
    const int osz = a.out_dtype == DT_FP8 ? 1 : 2;
    if (a.H % NW == 0 && (a.ldo * osz) % 16 == 0 && (reinterpret_cast<uintptr_t>(a.out) & 15) == 0) {
      if (a.out_dtype == DT_FP8) hipLaunchKernelGGL((attention_kernel<HS, MODE, 1, IN_DT, 1>), grid, block, 0, st, a);
      else if (a.out_dtype == IN_DT) hipLaunchKernelGGL((attention_kernel<HS, MODE, 0, IN_DT, 1>), grid, block, 0, st, a);
      else return hipErrorInvalidValue;
      return hipGetLastError();
    }
  }
  if (a.out_dtype == DT_FP8) hipLaunchKernelGGL((attention_kernel<HS, MODE, 1, IN_DT>), grid, block, 0, st, a);
  else if (a.out_dtype == IN_DT) hipLaunchKernelGGL((attention_kernel<HS, MODE, 0, IN_DT>), grid, block, 0, st, a);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

template <int HS, int MODE>
static hipError_t launch_attn_mode(const AttnArgs& a, hipStream_t st) {
  if (a.in_dtype == DT_F16) return launch_attn_dt<HS, MODE, DT_F16>(a, st);
  if (a.in_dtype == DT_BF16) return launch_attn_dt<HS, MODE, DT_BF16>(a, st);
  return hipErrorInvalidValue;
}

template <int HS>
static hipError_t launch_attn_hs(const AttnArgs& a, hipStream_t st) {
  switch (a.mode) {
    case ATTN_PLAIN: return launch_attn_mode<HS, ATTN_PLAIN>(a, st);
    case ATTN_CAUSAL: return launch_attn_mode<HS, ATTN_CAUSAL>(a, st);
    case ATTN_BIAS: return launch_attn_mode<HS, ATTN_BIAS>(a, st);
    case ATTN_RELSHIFT: return launch_attn_mode<HS, ATTN_RELSHIFT>(a, st);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_attention(const AttnArgs& a, int head_dim, hipStream_t st) {
  if (a.B <= 0) return hipSuccess;
  // 16-byte row-segment loads: strides and bases must be multiples of 8 elements.
  if (a.ldq % 8 || a.ldk % 8 || a.ldv % 8 || a.ldo % 4 || a.qk_hstride % 8 || (a.qk_hstride && (a.qk_hstride < head_dim || (a.T != 0 && a.T != 64))) ||
      (reinterpret_cast<uintptr_t>(a.q) & 15) || (reinterpret_cast<uintptr_t>(a.k) & 15) || (reinterpret_cast<uintptr_t>(a.v) & 15))
    return hipErrorInvalidValue;
  if (a.mode == ATTN_BIAS && !a.bias) return hipErrorInvalidValue;
  if (a.mode == ATTN_BIAS && a.bias_blocked && ((long)a.B * a.H) % 256 != 0) return hipErrorInvalidValue;
  if (a.mode == ATTN_RELSHIFT && (!a.pos || !a.u_bias || !a.v_bias)) return hipErrorInvalidValue;
  if (a.T != 0 && a.T != 64) {
    if (a.mode != ATTN_CAUSAL || a.T < 1 || a.T > 4096) return hipErrorInvalidValue;
    if (head_dim == 32) return launch_causal_long<32>(a, st);
    if (head_dim == 64) return launch_causal_long<64>(a, st);
    return hipErrorInvalidValue;
  }
  if (head_dim == 32) return launch_attn_hs<32>(a, st);
  if (head_dim == 64) return launch_attn_hs<64>(a, st);
  return hipErrorInvalidValue;
}

int attn_bias_slot_host(int i, int j) { return attn_bias_slot(i, j); }

}  // namespace crl
