// extern "C" surface declared in include/chessrl_amd.h.
#include <algorithm>
#include <cstring>
#include <thread>

#include "model.hpp"

using namespace crl;

namespace {

int hip_fail(const char* what, hipError_t e) {
  set_error(std::string(what) + ": " + hipGetErrorString(e));
  return CRL_ERR_HIP;
}
int arg_fail(const char* msg) {
  set_error(msg);
  return CRL_ERR_ARG;
}

// Run fn(i) for i in [0,n) on a few host threads; returns the first non-zero result.
template <typename Fn>
int parallel_for(int n, int threads, Fn fn) {
  if (threads <= 0) threads = (int)std::min<unsigned>(16, std::max<unsigned>(1, std::thread::hardware_concurrency()));
  threads = std::min(threads, std::max(1, n / 64));
  if (threads <= 1) {
    for (int i = 0; i < n; ++i) { int rc = fn(i); if (rc) return rc; }
    return 0;
  }
  std::vector<int> rcs(threads, 0);
  std::vector<std::string> errs(threads);
  std::vector<std::thread> pool;
  for (int t = 0; t < threads; ++t)
    pool.emplace_back([&, t]() {
      for (int i = t; i < n; i += threads) {
        int rc = fn(i);
        if (rc) { rcs[t] = rc; errs[t] = get_error(); return; }
      }
    });
  for (auto& th : pool) th.join();
  for (int t = 0; t < threads; ++t)
    if (rcs[t]) { set_error(errs[t]); return rcs[t]; }
  return 0;
}

int parse(const char* fen, Board& b) {
  std::string err;
  if (b.set_fen(fen, &err)) {
    set_error("invalid FEN '" + std::string(fen ? fen : "(null)") + "': " + err);
    return CRL_ERR_FEN;
  }
  return 0;
}

// Inverse move maps of crl_leela_to_rl on the device, one copy per device; crl_shutdown frees them.
int32_t* g_inv_dev[16] = {};

void put_str(char* dst, size_t cap, const std::string& s) {
  std::memset(dst, 0, cap);
  std::memcpy(dst, s.data(), std::min(cap - 1, s.size()));
}

}  // namespace

extern "C" {

const char* crl_last_error(void) { return get_error(); }
const char* crl_version(void) { return "chessrl_amd 0.2 (gfx950)"; }

void crl_shutdown(void) {
  release_gemm_globals();
  int cur = 0;
  const bool have_dev = hipGetDevice(&cur) == hipSuccess;
  for (int d = 0; d < 16; ++d)
    if (g_inv_dev[d]) {
      if (have_dev) (void)hipSetDevice(d);
      (void)hipFree(g_inv_dev[d]);
      g_inv_dev[d] = nullptr;
    }
  if (have_dev) (void)hipSetDevice(cur);
}

const char* crl_policy_index(int i) {
  const auto& v = policy_index();
  return (i >= 0 && i < (int)v.size()) ? v[i].c_str() : nullptr;
}
const char* crl_policy_leela(int i) {
  const auto& v = policy_leela();
  return (i >= 0 && i < (int)v.size()) ? v[i].c_str() : nullptr;
}
int crl_move_to_index(const char* uci) {
  if (!uci) return -1;
  std::string s = uci;
  if (s.size() == 5 && s[4] == 'n') s.pop_back();
  const auto& v = policy_index();
  for (int i = 0; i < (int)v.size(); ++i)
    if (v[i] == s) return i;
  return -1;
}
int crl_leela_to_rl_maps(int32_t* white_out, int32_t* black_out) {
  if (white_out) std::memcpy(white_out, leela_to_rl_white(), sizeof(int32_t) * VOCAB_LEELA);
  if (black_out) std::memcpy(black_out, leela_to_rl_black(), sizeof(int32_t) * VOCAB_LEELA);
  return CRL_OK;
}

int crl_fen_to_planes(const char* fen, float* out) {
  if (!out) return arg_fail("crl_fen_to_planes: null output");
  Board b;
  int rc = parse(fen, b);
  if (rc) return rc;
  b.planes(out);
  return CRL_OK;
}
int crl_encode_fens(const char* const* fens, int n, float* out, int threads) {
  if (n < 0 || (n && (!fens || !out))) return arg_fail("crl_encode_fens: bad arguments");
  return parallel_for(n, threads, [&](int i) {
    Board b;
    int rc = parse(fens[i], b);
    if (rc) return rc;
    b.planes(out + (size_t)i * 64 * NUM_PLANES);
    return 0;
  });
}
int crl_encode_fens_compact(const char* const* fens, int n, uint8_t* ids, uint8_t* flags, int threads) {
  if (n < 0 || (n && (!fens || !ids || !flags))) return arg_fail("crl_encode_fens_compact: bad arguments");
  return parallel_for(n, threads, [&](int i) {
    Board b;
    int rc = parse(fens[i], b);
    if (rc) return rc;
    b.compact(ids + (size_t)i * 64, flags + (size_t)i * 4);
    return 0;
  });
}
int crl_legal_masks(const char* const* fens, int n, uint8_t* masks, int32_t* counts, int threads) {
  if (n < 0 || (n && (!fens || !masks))) return arg_fail("crl_legal_masks: bad arguments");
  return parallel_for(n, threads, [&](int i) {
    Board b;
    int rc = parse(fens[i], b);
    if (rc) return rc;
    int c = legal_mask_rl(b, masks + (size_t)i * VOCAB_RL);
    if (counts) counts[i] = c;
    return 0;
  });
}
int crl_legal_masks_leela(const char* const* fens, int n, uint8_t* masks, int32_t* counts, int threads) {
  if (n < 0 || (n && (!fens || !masks))) return arg_fail("crl_legal_masks_leela: bad arguments");
  return parallel_for(n, threads, [&](int i) {
    Board b;
    int rc = parse(fens[i], b);
    if (rc) return rc;
    int c = legal_mask_leela(b, masks + (size_t)i * VOCAB_LEELA);
    if (counts) counts[i] = c;
    return 0;
  });
}
int crl_legal_moves(const char* fen, char* out_uci6, int max_moves) {
  Board b;
  int rc = parse(fen, b);
  if (rc) return rc;
  std::vector<Move> mv;
  b.legal(mv);
  const int n = std::min<int>((int)mv.size(), max_moves);
  for (int i = 0; i < n && out_uci6; ++i) put_str(out_uci6 + (size_t)i * 6, 6, move_uci(mv[i]));
  return n;
}
int crl_child_fens(const char* fen, char* out_fens96, char* out_uci6, int max_moves) {
  Board b;
  int rc = parse(fen, b);
  if (rc) return rc;
  std::vector<Move> mv;
  b.legal(mv);
  const int n = std::min<int>((int)mv.size(), max_moves);
  for (int i = 0; i < n; ++i) {
    Board c = b;
    c.make(mv[i]);
    if (out_fens96) put_str(out_fens96 + (size_t)i * 96, 96, c.fen(true));
    if (out_uci6) put_str(out_uci6 + (size_t)i * 6, 6, move_uci(mv[i]));
  }
  return n;
}
uint64_t crl_perft(const char* fen, int depth) {
  Board b;
  if (parse(fen, b)) return 0;
  return b.perft(depth);
}
int crl_random_positions(uint64_t seed, int n, int max_plies, double late_fraction, int late_max_pieces,
                         float* out_planes, uint8_t* out_masks_rl, uint8_t* out_masks_leela, char* out_fens96) {
  if (n < 0 || max_plies < 0) return arg_fail("crl_random_positions: bad arguments");
  // Every position has its own generator seeded from (seed, index), so the result does
  // not depend on the thread count.
  return parallel_for(n, 0, [&](int i) {
    SplitMix64 mix(seed ^ (0xD1B54A32D192ED03ull * (uint64_t)(i + 1)));
    SplitMix64 rng(mix.next());
    const bool late = late_fraction > 0 && (double)(rng.next() >> 11) * (1.0 / 9007199254740992.0) < late_fraction;
    Board b = random_playout(rng, max_plies, late ? late_max_pieces : 0);
    // Positions reach the models as FEN strings, and the FEN of a live board names the
    // en-passant square only when the capture is legal: encode what that FEN encodes.
    const std::string fen = b.fen(true);
    b.set_fen(fen.c_str());
    if (out_planes) b.planes(out_planes + (size_t)i * 64 * NUM_PLANES);
    if (out_masks_rl) legal_mask_rl(b, out_masks_rl + (size_t)i * VOCAB_RL);
    if (out_masks_leela) legal_mask_leela(b, out_masks_leela + (size_t)i * VOCAB_LEELA);
    if (out_fens96) put_str(out_fens96 + (size_t)i * 96, 96, fen);
    return 0;
  });
}

// ---------------------------------------------------------------------------- operators
int crl_gemm(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N, int K, int in_dtype,
             int out_dtype, const float* bias, int act, float descale, float alpha, const void* res, int64_t ldr, int res_dtype,
             float out_scale, float* amax, int tile, void* stream) {
  if (!A || !W || !C || M < 0 || N < 0 || K <= 0) return arg_fail("crl_gemm: bad arguments");
  if (in_dtype != DT_BF16 && in_dtype != DT_F16 && in_dtype != DT_FP8) return arg_fail("crl_gemm: in_dtype must be bf16, f16 or fp8");
  if (out_dtype < 0 || out_dtype > 3 || tile < 0 || tile > 16 || tile == 6 || tile == 8) return arg_fail("crl_gemm: bad out_dtype or tile");
  GemmArgs g;
  std::memset(&g, 0, sizeof(g));
  g.A = A; g.lda = lda; g.W = W; g.ldw = ldw; g.C = C; g.ldc = ldc; g.M = M; g.N = N; g.K = K; g.nsplit = N;
  g.bias = bias; g.act = act; g.descale = descale; g.alpha = alpha; g.res = res; g.ldr = ldr; g.res_dtype = res_dtype;
  g.out_scale = out_scale; g.amax = amax;
  hipError_t e = launch_gemm(g, in_dtype, out_dtype, tile, (hipStream_t)stream);
  if (e == hipErrorInvalidValue)
    return arg_fail("crl_gemm: operands must be 16-byte aligned with K*elem_size a multiple of 16");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_gemm", e);
}

int crl_gemm_split(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, void* C2, int64_t ldc2, int nsplit,
                   int M, int N, int K, int in_dtype, int out_dtype, const float* bias, float descale, int tile, void* stream) {
  if (!A || !W || !C || !C2 || M < 0 || N < 0 || K <= 0) return arg_fail("crl_gemm_split: bad arguments");
  if (nsplit <= 0 || nsplit >= N || nsplit % 8 != 0) return arg_fail("crl_gemm_split: nsplit must be a multiple of 8 inside (0, N)");
  if (in_dtype != DT_BF16 && in_dtype != DT_F16 && in_dtype != DT_FP8) return arg_fail("crl_gemm_split: in_dtype must be bf16, f16 or fp8");
  if (out_dtype < 0 || out_dtype > 3 || (tile != 0 && tile != 3 && tile != 7 && tile != 10)) return arg_fail("crl_gemm_split: bad out_dtype or tile");
  GemmArgs g;
  std::memset(&g, 0, sizeof(g));
  g.A = A; g.lda = lda; g.W = W; g.ldw = ldw; g.C = C; g.ldc = ldc; g.C2 = C2; g.ldc2 = ldc2; g.M = M; g.N = N; g.K = K; g.nsplit = nsplit;
  g.bias = bias; g.descale = descale; g.alpha = 1.f; g.out_scale = 1.f;
  hipError_t e = launch_gemm(g, in_dtype, out_dtype, tile, (hipStream_t)stream);
  if (e == hipErrorInvalidValue)
    return arg_fail("crl_gemm_split: operands must be 16-byte aligned with K*elem_size a multiple of 16");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_gemm_split", e);
}

int crl_gemm_static_scratch(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N, int K, int in_dtype,
                            int out_dtype, const float* bias, int act, float descale, float alpha, const void* res, int64_t ldr,
                            int res_dtype, float out_scale, float* amax, void* stream) {
  if (!A || !W || !C || M < 0 || N < 0 || K <= 0) return arg_fail("crl_gemm_static_scratch: bad arguments");
  if (in_dtype != DT_BF16 && in_dtype != DT_F16 && in_dtype != DT_FP8) return arg_fail("crl_gemm_static_scratch: in_dtype must be bf16, f16 or fp8");
  if (out_dtype < 0 || out_dtype > 3) return arg_fail("crl_gemm_static_scratch: bad out_dtype");
  GemmArgs g;
  std::memset(&g, 0, sizeof(g));
  g.A = A; g.lda = lda; g.W = W; g.ldw = ldw; g.C = C; g.ldc = ldc; g.M = M; g.N = N; g.K = K; g.nsplit = N;
  g.bias = bias; g.act = act; g.descale = descale; g.alpha = alpha; g.res = res; g.ldr = ldr; g.res_dtype = res_dtype;
  g.out_scale = out_scale; g.amax = amax;
  bool too_big = false;
  size_t need = 0;
  hipError_t e = launch_gemm_static_ws(g, in_dtype, out_dtype, (hipStream_t)stream, &too_big, &need);
  if (too_big) {
    set_error("crl_gemm_static_scratch: the K slices of this product need " + std::to_string(need) + " bytes of partial sums, the fixed scratch array holds " +
              std::to_string((size_t)STATIC_WS_BYTES) + " (use crl_gemm, which allocates)");
    return CRL_ERR_ARG;
  }
  if (e == hipErrorInvalidValue)
    return arg_fail("crl_gemm_static_scratch: operands must be 16-byte aligned with K*elem_size a multiple of 16");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_gemm_static_scratch", e);
}
int64_t crl_gemm_static_scratch_bytes(void) { return (int64_t)STATIC_WS_BYTES; }

int crl_layernorm(const void* x, int64_t ldx, int in_dtype, const float* gamma, const float* beta, void* out, int out_dtype,
                  uint8_t* out_fp8, float fp8_scale, int64_t ldo, int rows, int C, float eps, float* amax, void* stream) {
  if (!x || !gamma || (!out && !out_fp8) || rows < 0) return arg_fail("crl_layernorm: bad arguments");
  LayerNormArgs a;
  std::memset(&a, 0, sizeof(a));
  a.x = x; a.ldx = ldx; a.in_dtype = in_dtype; a.gamma = gamma; a.beta = beta; a.out = out; a.out_dtype = out_dtype;
  a.out_fp8 = out_fp8; a.fp8_scale = fp8_scale; a.ldo = ldo; a.rows = rows; a.C = C; a.eps = eps; a.amax = amax;
  hipError_t e = launch_layernorm(a, (hipStream_t)stream);
  if (e == hipErrorInvalidValue) return arg_fail("crl_layernorm: C and strides must be multiples of 8 and C <= 8192");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_layernorm", e);
}

int crl_rmsnorm(const void* x, int64_t ldx, int in_dtype, const float* gamma, void* out, int out_dtype, uint8_t* out_fp8, float fp8_scale,
                int64_t ldo, int rows, int C, float eps, float* amax, void* stream) {
  if (!x || !gamma || (!out && !out_fp8) || rows < 0) return arg_fail("crl_rmsnorm: bad arguments");
  LayerNormArgs a;
  std::memset(&a, 0, sizeof(a));
  a.x = x; a.ldx = ldx; a.in_dtype = in_dtype; a.gamma = gamma; a.out = out; a.out_dtype = out_dtype;
  a.out_fp8 = out_fp8; a.fp8_scale = fp8_scale; a.ldo = ldo; a.rows = rows; a.C = C; a.eps = eps; a.amax = amax; a.rms = 1;
  hipError_t e = launch_layernorm(a, (hipStream_t)stream);
  if (e == hipErrorInvalidValue) return arg_fail("crl_rmsnorm: C and strides must be multiples of 8 and C <= 8192");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_rmsnorm", e);
}

int crl_attention(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v, int64_t ldv, int in_dtype, void* out, int64_t ldo,
                  int out_dtype, float out_scale, int B, int H, int head_dim, int mode, float scale, const void* bias,
                  const void* pos, const float* u_bias, const float* v_bias, float* amax, void* stream) {
  if (!q || !k || !v || !out || B < 0 || H <= 0) return arg_fail("crl_attention: bad arguments");
  AttnArgs a;
  std::memset(&a, 0, sizeof(a));
  a.q = q; a.k = k; a.v = v; a.ldq = ldq; a.ldk = ldk; a.ldv = ldv; a.in_dtype = in_dtype; a.out = out; a.ldo = ldo; a.out_dtype = out_dtype;
  a.out_scale = out_scale; a.B = B; a.H = H; a.mode = mode; a.scale = scale; a.bias = bias; a.pos = pos;
  a.u_bias = u_bias; a.v_bias = v_bias; a.amax = amax;
  hipError_t e = launch_attention(a, head_dim, (hipStream_t)stream);
  if (e == hipErrorInvalidValue) return arg_fail("crl_attention: head_dim must be 32 or 64, in_dtype bf16/f16, out_dtype in_dtype or fp8, strides multiples of 8, mode inputs present");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_attention", e);
}

int crl_attn_bias_slot(int query, int key) {
  if (query < 0 || query > 63 || key < 0 || key > 63) return -1;
  return attn_bias_slot_host(query, key);
}

int crl_masked_softmax(const float* logits, int64_t ldl, const uint8_t* mask, int64_t ldm, float* probs, int64_t ldp,
                       int32_t* argmax, int B, int V, float temperature, void* stream) {
  if (!logits || B < 0) return arg_fail("crl_masked_softmax: bad arguments");
  SoftmaxArgs a;
  std::memset(&a, 0, sizeof(a));
  a.logits = logits; a.ldl = ldl; a.mask = mask; a.ldm = ldm; a.probs = probs; a.ldp = ldp; a.argmax = argmax;
  a.B = B; a.V = V; a.temperature = temperature;
  hipError_t e = launch_masked_softmax(a, (hipStream_t)stream);
  if (e == hipErrorInvalidValue) return arg_fail("crl_masked_softmax: V must be in 1..2048");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_masked_softmax", e);
}

int crl_leela_to_rl(const float* src, int64_t lds, float* dst, int64_t ldd, const uint8_t* white_to_move, int B, void* stream) {
  if (!src || !dst || !white_to_move || B < 0) return arg_fail("crl_leela_to_rl: bad arguments");
  // Inverse maps live on the device for the lifetime of the process, one copy per device.
  int32_t** inv_dev = g_inv_dev;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail("hipGetDevice", e);
  if (dev < 0 || dev >= 16) return arg_fail("crl_leela_to_rl: device index above 15");
  if (!inv_dev[dev]) {
    std::vector<int32_t> inv((size_t)2 * VOCAB_RL, -1);
    for (int i = 0; i < VOCAB_LEELA; ++i) {
      inv[leela_to_rl_white()[i]] = i;
      inv[VOCAB_RL + leela_to_rl_black()[i]] = i;
    }
    int32_t* p = nullptr;
    e = hipMalloc((void**)&p, inv.size() * sizeof(int32_t));
    if (e != hipSuccess) return hip_fail("hipMalloc", e);
    e = hipMemcpy(p, inv.data(), inv.size() * sizeof(int32_t), hipMemcpyHostToDevice);
    if (e != hipSuccess) { (void)hipFree(p); return hip_fail("hipMemcpy", e); }
    inv_dev[dev] = p;
  }
  ScatterArgs a;
  std::memset(&a, 0, sizeof(a));
  a.src = src; a.lds = lds; a.dst = dst; a.ldd = ldd; a.inv_white = inv_dev[dev]; a.inv_black = inv_dev[dev] + VOCAB_RL;
  a.white_to_move = white_to_move; a.B = B; a.nsrc = VOCAB_LEELA; a.ndst = VOCAB_RL;
  e = launch_leela_to_rl(a, (hipStream_t)stream);
  return e == hipSuccess ? CRL_OK : hip_fail("crl_leela_to_rl", e);
}

int crl_attention_causal(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v, int64_t ldv, int in_dtype, void* out,
                         int64_t ldo, int out_dtype, float out_scale, int B, int H, int head_dim, int T, float scale, float* amax, void* stream) {
  if (!q || !k || !v || !out || B < 0 || H <= 0 || T < 1) return arg_fail("crl_attention_causal: bad arguments");
  AttnArgs a;
  std::memset(&a, 0, sizeof(a));
  a.q = q; a.k = k; a.v = v; a.ldq = ldq; a.ldk = ldk; a.ldv = ldv; a.in_dtype = in_dtype; a.out = out; a.ldo = ldo;
  a.out_dtype = out_dtype; a.out_scale = out_scale; a.B = B; a.H = H; a.mode = ATTN_CAUSAL; a.scale = scale; a.amax = amax;
  a.T = T == 64 ? 0 : T;
  hipError_t e = launch_attention(a, head_dim, (hipStream_t)stream);
  if (e == hipErrorInvalidValue) return arg_fail("crl_attention_causal: head_dim must be 32 or 64, in_dtype bf16/f16, out_dtype in_dtype or fp8, strides multiples of 8, T <= 4096");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_attention_causal", e);
}
int crl_sample(const float* logits, int64_t ldl, int B, int V, float temperature, uint64_t seed, int step, int64_t* tokens, float* probs,
               void* stream) {
  if (!logits || !tokens || B < 0 || V <= 0 || V > 2048 || temperature < 0.f) return arg_fail("crl_sample: bad arguments (V <= 2048)");
  SampleArgs a;
  std::memset(&a, 0, sizeof(a));
  a.logits = logits; a.ldl = ldl; a.seq = tokens; a.ld_seq = 1; a.tok_out = tokens; a.step_out = probs; a.ld_out = V;
  a.B = B; a.V = V; a.k = 0; a.step = step; a.temperature = temperature; a.seed = seed;
  hipError_t e = launch_sample(a, (hipStream_t)stream);
  return e == hipSuccess ? CRL_OK : hip_fail("crl_sample", e);
}
int crl_token_scores(const float* logits, int64_t ldl, const float* ref_logits, int64_t ldr, const int64_t* target, int rows, int V,
                     int64_t ignore_index, float* logp, float* ref_logp, float* kl, void* stream) {
  if (!logits || rows < 0 || V <= 0) return arg_fail("crl_token_scores: bad arguments");
  if (V > 2048) return arg_fail("crl_token_scores: at most 2048 classes");
  if ((kl || ref_logp) && !ref_logits) return arg_fail("crl_token_scores: reference logits missing");
  if ((logp || ref_logp) && !target) return arg_fail("crl_token_scores: targets missing");
  TokenScoreArgs a;
  std::memset(&a, 0, sizeof(a));
  a.logits = logits; a.ldl = ldl; a.ref = ref_logits; a.ldr = ldr; a.target = target; a.rows = rows; a.V = V;
  a.ignore_index = ignore_index; a.logp = logp; a.ref_logp = ref_logp; a.kl = kl;
  hipError_t e = launch_token_scores(a, (hipStream_t)stream);
  return e == hipSuccess ? CRL_OK : hip_fail("crl_token_scores", e);
}
int crl_masked_nll_mean(const float* logp, const int64_t* target, int64_t ignore_index, int rows, float* out, void* stream) {
  if (!logp || !target || !out || rows < 0) return arg_fail("crl_masked_nll_mean: bad arguments");
  hipError_t e = launch_masked_nll_mean(logp, target, ignore_index, rows, out, (hipStream_t)stream);
  return e == hipSuccess ? CRL_OK : hip_fail("crl_masked_nll_mean", e);
}

// ---------------------------------------------------------------------------- models
// Double-buffered staging of the FEN front-end: pinned host and device buffers for two chunks,
// one copy stream, one compute stream (both default priority), events per slot.
struct FenPipeline {
  int chunk = 0, vocab = 0;
  hipStream_t copy_st = nullptr, comp_st = nullptr;
  struct Slot {
    uint8_t *h_ids = nullptr, *h_flags = nullptr, *h_mask = nullptr;  // pinned inputs
    float *h_probs = nullptr, *h_wdl = nullptr; int32_t* h_best = nullptr;  // pinned outputs
    uint8_t *d_ids = nullptr, *d_flags = nullptr, *d_mask = nullptr;
    float *d_logits = nullptr, *d_probs = nullptr, *d_wdl = nullptr; int32_t* d_best = nullptr;
    hipEvent_t uploaded = nullptr, done = nullptr;
    int first = 0, count = 0;  // positions of the chunk in flight (count 0 = idle)
  } slot[2];
  void release() {
    for (Slot& s : slot) {
      (void)hipHostFree(s.h_ids); (void)hipHostFree(s.h_flags); (void)hipHostFree(s.h_mask);
      (void)hipHostFree(s.h_probs); (void)hipHostFree(s.h_wdl); (void)hipHostFree(s.h_best);
      (void)hipFree(s.d_ids); (void)hipFree(s.d_flags); (void)hipFree(s.d_mask);
      (void)hipFree(s.d_logits); (void)hipFree(s.d_probs); (void)hipFree(s.d_wdl); (void)hipFree(s.d_best);
      if (s.uploaded) (void)hipEventDestroy(s.uploaded);
      if (s.done) (void)hipEventDestroy(s.done);
      s = Slot();
    }
    if (copy_st) (void)hipStreamDestroy(copy_st);
    if (comp_st) (void)hipStreamDestroy(comp_st);
    copy_st = comp_st = nullptr;
    chunk = 0;
  }
  hipError_t ensure(int want_chunk, int V) {
    if (want_chunk <= chunk && V == vocab) return hipSuccess;
    release();
    hipError_t e;
#define PIPE_TRY(call) do { e = (call); if (e != hipSuccess) { release(); return e; } } while (0)
    PIPE_TRY(hipStreamCreateWithFlags(&copy_st, hipStreamNonBlocking));
    PIPE_TRY(hipStreamCreateWithFlags(&comp_st, hipStreamNonBlocking));
    const size_t c = (size_t)want_chunk;
    for (Slot& s : slot) {
      PIPE_TRY(hipHostMalloc((void**)&s.h_ids, c * 64, hipHostMallocDefault));
      PIPE_TRY(hipHostMalloc((void**)&s.h_flags, c * 4, hipHostMallocDefault));
      PIPE_TRY(hipHostMalloc((void**)&s.h_mask, c * V, hipHostMallocDefault));
      PIPE_TRY(hipHostMalloc((void**)&s.h_probs, c * V * sizeof(float), hipHostMallocDefault));
      PIPE_TRY(hipHostMalloc((void**)&s.h_wdl, c * 3 * sizeof(float), hipHostMallocDefault));
      PIPE_TRY(hipHostMalloc((void**)&s.h_best, c * sizeof(int32_t), hipHostMallocDefault));
      PIPE_TRY(hipMalloc((void**)&s.d_ids, c * 64));
      PIPE_TRY(hipMalloc((void**)&s.d_flags, c * 4));
      PIPE_TRY(hipMalloc((void**)&s.d_mask, c * V));
      PIPE_TRY(hipMalloc((void**)&s.d_logits, c * V * sizeof(float)));
      PIPE_TRY(hipMalloc((void**)&s.d_probs, c * V * sizeof(float)));
      PIPE_TRY(hipMalloc((void**)&s.d_wdl, c * 3 * sizeof(float)));
      PIPE_TRY(hipMalloc((void**)&s.d_best, c * sizeof(int32_t)));
      PIPE_TRY(hipEventCreateWithFlags(&s.uploaded, hipEventDisableTiming));
      PIPE_TRY(hipEventCreateWithFlags(&s.done, hipEventDisableTiming));
    }
#undef PIPE_TRY
    chunk = want_chunk; vocab = V;
    return hipSuccess;
  }
};

struct crl_model {
  Model impl;
  FenPipeline pipe;
  explicit crl_model(const crl_model_config& c) : impl(c) {}
  ~crl_model() { pipe.release(); }
};

int crl_model_create(const crl_model_config* cfg, crl_model** out) {
  if (!cfg || !out) return arg_fail("crl_model_create: null argument");
  if (cfg->arch < 0 || cfg->arch > 2) return arg_fail("crl_model_create: unknown arch");
  if (cfg->n_layer < 0 || cfg->d_model <= 0 || cfg->n_head <= 0 || cfg->d_ff <= 0) return arg_fail("crl_model_create: non-positive size");
  if (cfg->d_model % cfg->n_head) return arg_fail("crl_model_create: d_model must be divisible by n_head");
  const int hs = cfg->d_model / cfg->n_head;
  if (hs != 32 && hs != 64) return arg_fail("crl_model_create: head dimension must be 32 or 64");
  if (cfg->d_model % 16 || cfg->d_model > 2048 || cfg->d_ff % 8) return arg_fail("crl_model_create: d_model must be a multiple of 16 up to 2048, d_ff a multiple of 8");
  if (cfg->arch != CRL_ARCH_GPT64 && cfg->d_model % 64)
    return arg_fail("crl_model_create: d_model must be a multiple of 64 for CRL_ARCH_BT4 and CRL_ARCH_BT4CLASS (the policy head's product splits the channels over four waves in steps of 16)");
  if (cfg->arch == CRL_ARCH_BT4CLASS) {
    const int sg = cfg->smolgen_gen ? cfg->smolgen_gen : 256, sc = cfg->smolgen_compress ? cfg->smolgen_compress : 32;
    const int sh = cfg->smolgen_hidden ? cfg->smolgen_hidden : 256;
    if (sg % 8 || sc % 8 || sh % 8 || (long)cfg->n_head * sg > 8192) return arg_fail("crl_model_create: smolgen sizes must be multiples of 8 and n_head*gen <= 8192");
  }
  *out = new (std::nothrow) crl_model(*cfg);
  if (!*out) return arg_fail("crl_model_create: out of host memory");
  return CRL_OK;
}
void crl_model_destroy(crl_model* m) { delete m; }
int crl_model_set_weight(crl_model* m, const char* key, const float* data, int64_t numel) {
  if (!m) return arg_fail("null model");
  return m->impl.set_weight(key, data, (long)numel);
}
const char* crl_model_expected_key(crl_model* m, int i, int64_t* numel) {
  if (!m || i < 0 || i >= (int)m->impl.expected.size()) return nullptr;
  if (numel) *numel = m->impl.expected[i].second;
  return m->impl.expected[i].first.c_str();
}
int crl_model_finalize(crl_model* m) {
  if (!m) return arg_fail("null model");
  return m->impl.finalize();
}
int crl_model_calibrate(crl_model* m, const float* planes, int B, void* stream) {
  if (!m || !planes || B <= 0) return arg_fail("crl_model_calibrate: bad arguments");
  return m->impl.calibrate(planes, B, (hipStream_t)stream);
}
int crl_model_get_amax(crl_model* m, float* out, int n) {
  if (!m) return arg_fail("crl_model_get_amax: null model");
  const int full = (int)m->impl.amax_host.size();   // (n_layer + 1) * 5
  if (!m || !out || (n != full && n != full - Model::AMAX_SLOTS)) return arg_fail("crl_model_get_amax: n must be n_layer*5 or (n_layer+1)*5");
  std::memcpy(out, m->impl.amax_host.data(), sizeof(float) * n);
  return CRL_OK;
}
int crl_model_set_amax(crl_model* m, const float* in, int n) {
  if (!m) return arg_fail("crl_model_set_amax: null model");
  const int full = (int)m->impl.amax_host.size();
  if (!m || !in || (n != full && n != full - Model::AMAX_SLOTS)) return arg_fail("crl_model_set_amax: n must be n_layer*5 or (n_layer+1)*5");
  std::memcpy(m->impl.amax_host.data(), in, sizeof(float) * n);
  return CRL_OK;
}
int crl_model_forward(crl_model* m, const float* planes, int B, float* policy_logits, float* wdl_logits, void* stream) {
  if (m && B == 0) return CRL_OK;  // an empty batch writes nothing (its buffers may be null)
  if (!m || !planes) return arg_fail("crl_model_forward: bad arguments");
  return m->impl.forward(planes, nullptr, nullptr, B, policy_logits, wdl_logits, false, (hipStream_t)stream);
}
int crl_model_forward_compact(crl_model* m, const uint8_t* ids, const uint8_t* flags, int B, float* policy_logits,
                              float* wdl_logits, void* stream) {
  if (m && B == 0) return CRL_OK;
  if (!m || !ids || !flags) return arg_fail("crl_model_forward_compact: bad arguments");
  return m->impl.forward(nullptr, ids, flags, B, policy_logits, wdl_logits, false, (hipStream_t)stream);
}
int crl_model_forward_tokens(crl_model* m, const float* planes, const int64_t* idx, int B, int t, float* last_logits,
                             float* all_logits, void* stream) {
  if (m && B == 0) return CRL_OK;
  if (!m || !planes) return arg_fail("crl_model_forward_tokens: bad arguments");
  return m->impl.forward_tokens(planes, nullptr, nullptr, idx, t, B, last_logits, all_logits, nullptr, false, (hipStream_t)stream);
}
int crl_model_generate(crl_model* m, const float* planes, int B, int steps, float temperature, uint64_t seed, int rules,
                       int64_t* sequences, float* step_out, int out_logits, void* stream) {
  if (!m) return arg_fail("crl_model_generate: null model");
  return m->impl.generate(planes, B, steps, temperature, seed, rules, sequences, step_out, out_logits, (hipStream_t)stream);
}
}  // extern "C"

// The chunked host -> device -> host pipeline behind crl_model_evaluate_fens and crl_model_search_1ply: position i of
// the job is produced by get(i, board) on the host threads. The legal-move masks and the masked softmax are skipped
// when neither probabilities nor best moves are asked for (value-only evaluation).
template <typename GetBoard>
static int evaluate_boards(crl_model* m, int n, int chunk, float temperature, float* probs, float* wdl, int32_t* best, int threads,
                           GetBoard get) {
  const int V = m->impl.vocab;
  const bool leela = m->impl.cfg.arch == CRL_ARCH_BT4CLASS, has_wdl = m->impl.cfg.arch != CRL_ARCH_GPT64;
  const bool need_policy = probs || best;
  if (n == 0) return CRL_OK;
  if (chunk > n) chunk = n;
  FenPipeline& P = m->pipe;
  // The pipeline runs on streams of its own and shares the model's workspace with every other entry point: work a
  // caller has queued on this model through crl_model_forward (on any stream) must have finished before the first
  // chunk starts, and the workspace may be re-allocated below. Nothing here knows the caller's streams, so wait for
  // the device.
  hipError_t e = hipDeviceSynchronize();
  if (e != hipSuccess) return hip_fail("evaluate: waiting for earlier work on the device", e);
  e = P.ensure(chunk, V);
  if (e != hipSuccess) return hip_fail("evaluate: staging buffers", e);
  // Results of a finished slot go from pinned staging to the caller's arrays.
  auto drain = [&](FenPipeline::Slot& s) -> hipError_t {
    if (s.count == 0) return hipSuccess;
    hipError_t de = hipEventSynchronize(s.done);
    if (de != hipSuccess) return de;
    if (probs) std::memcpy(probs + (size_t)s.first * V, s.h_probs, sizeof(float) * (size_t)s.count * V);
    if (wdl) std::memcpy(wdl + (size_t)s.first * 3, s.h_wdl, sizeof(float) * (size_t)s.count * 3);
    if (best) std::memcpy(best + s.first, s.h_best, sizeof(int32_t) * (size_t)s.count);
    s.count = 0;
    return hipSuccess;
  };
  int rc = CRL_OK;
  int k = 0;
  for (int first = 0; first < n && rc == CRL_OK; first += chunk, ++k) {
    FenPipeline::Slot& s = P.slot[k & 1];
    e = drain(s);  // the chunk that used this slot two steps ago
    if (e != hipSuccess) { rc = hip_fail("evaluate: wait", e); break; }
    const int cnt = std::min(chunk, n - first);
    // Host work of this chunk overlaps the device work of the previous one.
    rc = parallel_for(cnt, threads, [&](int i) {
      Board b;
      int prc = get(first + i, b);
      if (prc) return prc;
      b.compact(s.h_ids + (size_t)i * 64, s.h_flags + (size_t)i * 4);
      if (!need_policy) return 0;
      if (leela) legal_mask_leela(b, s.h_mask + (size_t)i * V);
      else legal_mask_rl(b, s.h_mask + (size_t)i * V);
      return 0;
    });
    if (rc) break;
#define PIPE_HIP(call) do { e = (call); if (e != hipSuccess) { rc = hip_fail("evaluate", e); } } while (0)
    PIPE_HIP(hipMemcpyAsync(s.d_ids, s.h_ids, (size_t)cnt * 64, hipMemcpyHostToDevice, P.copy_st));
    if (rc == CRL_OK) PIPE_HIP(hipMemcpyAsync(s.d_flags, s.h_flags, (size_t)cnt * 4, hipMemcpyHostToDevice, P.copy_st));
    if (rc == CRL_OK && need_policy) PIPE_HIP(hipMemcpyAsync(s.d_mask, s.h_mask, (size_t)cnt * V, hipMemcpyHostToDevice, P.copy_st));
    if (rc == CRL_OK) PIPE_HIP(hipEventRecord(s.uploaded, P.copy_st));
    if (rc == CRL_OK) PIPE_HIP(hipStreamWaitEvent(P.comp_st, s.uploaded, 0));
    if (rc) break;
    rc = m->impl.forward(nullptr, s.d_ids, s.d_flags, cnt, s.d_logits, has_wdl ? s.d_wdl : nullptr, false, P.comp_st);
    if (rc) break;
    if (need_policy) {
      SoftmaxArgs a;
      std::memset(&a, 0, sizeof(a));
      a.logits = s.d_logits; a.ldl = V; a.mask = s.d_mask; a.ldm = V; a.probs = probs ? s.d_probs : nullptr; a.ldp = V;
      a.argmax = s.d_best; a.B = cnt; a.V = V; a.temperature = temperature;
      PIPE_HIP(launch_masked_softmax(a, P.comp_st));
    }
    if (rc == CRL_OK && probs) PIPE_HIP(hipMemcpyAsync(s.h_probs, s.d_probs, sizeof(float) * (size_t)cnt * V, hipMemcpyDeviceToHost, P.comp_st));
    if (rc == CRL_OK && wdl) PIPE_HIP(hipMemcpyAsync(s.h_wdl, s.d_wdl, sizeof(float) * (size_t)cnt * 3, hipMemcpyDeviceToHost, P.comp_st));
    if (rc == CRL_OK && best) PIPE_HIP(hipMemcpyAsync(s.h_best, s.d_best, sizeof(int32_t) * (size_t)cnt, hipMemcpyDeviceToHost, P.comp_st));
    if (rc == CRL_OK) PIPE_HIP(hipEventRecord(s.done, P.comp_st));
#undef PIPE_HIP
    if (rc == CRL_OK) { s.first = first; s.count = cnt; }
  }
  // Leave nothing in flight, also on an error path (the staging buffers are reused by the next call).
  const std::string err = rc ? std::string(get_error()) : std::string();
  for (FenPipeline::Slot& s : P.slot) {
    if (rc == CRL_OK) {
      e = drain(s);
      if (e != hipSuccess) rc = hip_fail("evaluate: wait", e);
    } else {
      s.count = 0;
    }
  }
  if (rc != CRL_OK) {
    (void)hipStreamSynchronize(P.copy_st);
    (void)hipStreamSynchronize(P.comp_st);
    if (!err.empty()) set_error(err);
  }
  return rc;
}
extern "C" {

int crl_model_evaluate_fens(crl_model* m, const char* const* fens, int n, int chunk, float temperature, float* probs,
                            float* wdl, int32_t* best, int threads) {
  if (!m || n < 0 || (n && !fens) || chunk <= 0) return arg_fail("crl_model_evaluate_fens: bad arguments");
  if (!m->impl.finalized) { set_error("crl_model_evaluate_fens: call crl_model_finalize first"); return CRL_ERR_STATE; }
  if (wdl && m->impl.cfg.arch == CRL_ARCH_GPT64) return arg_fail("crl_model_evaluate_fens: this architecture has no value head");
  return evaluate_boards(m, n, chunk, temperature, probs, wdl, best, threads, [&](int i, Board& b) { return parse(fens[i], b); });
}

int crl_model_search_1ply(crl_model* m, const char* const* fens, int n, int chunk, float temperature, uint64_t seed, char* best_uci6,
                          int32_t* n_moves, char* moves_uci6, float* values, int64_t capacity, int threads) {
  if (!m || n < 0 || (n && !fens) || chunk <= 0 || temperature < 0.f || capacity < 0)
    return arg_fail("crl_model_search_1ply: bad arguments");
  if (!m->impl.finalized) { set_error("crl_model_search_1ply: call crl_model_finalize first"); return CRL_ERR_STATE; }
  if (m->impl.cfg.arch == CRL_ARCH_GPT64) return arg_fail("crl_model_search_1ply: this architecture has no value head");
  // Roots -> children on the host threads.
  std::vector<Board> roots(n);
  std::vector<std::vector<Move>> moves(n);
  int rc = parallel_for(n, threads, [&](int i) {
    int prc = parse(fens[i], roots[i]);
    if (prc) return prc;
    roots[i].legal(moves[i]);
    return 0;
  });
  if (rc) return rc;
  std::vector<int64_t> first(n + 1, 0);
  for (int i = 0; i < n; ++i) first[i + 1] = first[i] + (int64_t)moves[i].size();
  const int64_t total = first[n];
  if ((moves_uci6 || values) && total > capacity) {
    set_error("crl_model_search_1ply: " + std::to_string(total) + " child positions, room for " + std::to_string(capacity));
    return CRL_ERR_ARG;
  }
  if (total > INT32_MAX) return arg_fail("crl_model_search_1ply: too many child positions for one call");
  std::vector<int32_t> root_of((size_t)total);
  for (int i = 0; i < n; ++i)
    for (int64_t c = first[i]; c < first[i + 1]; ++c) root_of[(size_t)c] = i;
  std::vector<float> wdl((size_t)total * 3);
  rc = evaluate_boards(m, (int)total, chunk, 1.0f, nullptr, wdl.data(), nullptr, threads, [&](int c, Board& b) {
    // board.push(move); board.fen() and back (value.py:336-340, 288): the en-passant square survives only where a
    // capture is legal, which is what the planes of the child position are then built from.
    const int i = root_of[(size_t)c];
    Board child = roots[i];
    child.make(moves[i][(size_t)(c - first[i])]);
    return parse(child.fen(true).c_str(), b);
  });
  if (rc) return rc;
  // Per root: value of each child for the side to move at the root, then the pick (value.py:343-352, 372-395).
  for (int i = 0; i < n; ++i) {
    const int nm = (int)moves[i].size();
    if (n_moves) n_moves[i] = nm;
    if (best_uci6) std::memset(best_uci6 + (size_t)i * 6, 0, 6);
    if (nm == 0) continue;
    std::vector<float> val((size_t)nm);
    for (int c = 0; c < nm; ++c) {
      const float* w = wdl.data() + (size_t)(first[i] + c) * 3;
      const float mx = std::max(w[0], std::max(w[1], w[2]));
      const float e0 = std::exp(w[0] - mx), e1 = std::exp(w[1] - mx), e2 = std::exp(w[2] - mx);
      const float inv = 1.0f / (e0 + e1 + e2);
      val[(size_t)c] = 0.5f * e1 * inv + (roots[i].white_to_move ? e2 : e0) * inv;
      if (values) values[first[i] + c] = val[(size_t)c];
      if (moves_uci6) put_str(moves_uci6 + (size_t)(first[i] + c) * 6, 6, move_uci(moves[i][(size_t)c]));
    }
    int pick = 0;
    for (int c = 1; c < nm; ++c)
      if (val[(size_t)c] > val[(size_t)pick]) pick = c;
    if (temperature > 0.f) {
      // one draw from softmax(values / T): inverse CDF with a generator keyed by (seed, root)
      double sum = 0.0;
      std::vector<double> p((size_t)nm);
      for (int c = 0; c < nm; ++c) { p[(size_t)c] = std::exp((double)(val[(size_t)c] - val[(size_t)pick]) / temperature); sum += p[(size_t)c]; }
      SplitMix64 rng(seed ^ (0x9E3779B97F4A7C15ull * (uint64_t)(i + 1)));
      const double u = (double)(rng.next() >> 11) * (1.0 / 9007199254740992.0) * sum;
      double acc = 0.0;
      int drawn = nm - 1;
      for (int c = 0; c < nm; ++c) { acc += p[(size_t)c]; if (u < acc) { drawn = c; break; } }
      pick = drawn;
    }
    if (best_uci6) put_str(best_uci6 + (size_t)i * 6, 6, move_uci(moves[i][(size_t)pick]));
  }
  return CRL_OK;
}
int crl_model_run_layers(crl_model* m, const float* x_in, int B, int first, int last, float* x_out, void* stream) {
  if (!m) return arg_fail("crl_model_run_layers: null model");
  return m->impl.run_layers(x_in, B, first, last, x_out, (hipStream_t)stream);
}
int crl_model_read_tensor(crl_model* m, const char* name, void* out, int64_t bytes, void* stream) {
  if (!m) return arg_fail("crl_model_read_tensor: null model");
  return m->impl.debug_read(name, out, (long)bytes, (hipStream_t)stream);
}
int crl_model_vocab(const crl_model* m) { return m ? m->impl.vocab : 0; }
double crl_model_flops_per_position(const crl_model* m) { return m ? m->impl.flops_per_position() : 0.0; }
int crl_model_set_profiling(crl_model* m, int on) {
  if (!m) return arg_fail("null model");
  m->impl.profiling = on != 0;
  for (int i = 0; i < 6; ++i) { m->impl.prof_ms[i] = 0; m->impl.prof_n[i] = 0; m->impl.prof_flops[i] = 0; }
  return CRL_OK;
}
int crl_model_set_decode_graph(crl_model* m, int on) {
  if (!m) return arg_fail("null model");
  m->impl.decode_graph = on != 0;
  return CRL_OK;
}
int crl_model_get_profile(crl_model* m, double* ms6, int64_t* launches6, double* flops6) {
  if (!m || !ms6 || !launches6) return arg_fail("crl_model_get_profile: bad arguments");
  for (int i = 0; i < 6; ++i) {
    ms6[i] = m->impl.prof_ms[i];
    launches6[i] = m->impl.prof_n[i];
    if (flops6) flops6[i] = m->impl.prof_flops[i];
  }
  return CRL_OK;
}

int crl_probe_mfma(int dtype, int random_bits, int iters, double* tflops, double* ghz, void* stream) {
  if ((dtype != DT_BF16 && dtype != DT_F16 && dtype != DT_FP8) || iters <= 0 || !tflops || !ghz) return arg_fail("crl_probe_mfma: bad arguments");
  hipError_t e = run_mfma_probe(dtype, random_bits, iters, tflops, ghz, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail("crl_probe_mfma", e);
  return CRL_OK;
}

int crl_probe_cu_split(int gemm_cus, int tile, int rows, int iters, double* out8) {
  if (!out8) return arg_fail("crl_probe_cu_split: null output");
  if (tile < 0 || tile > 14) return arg_fail("crl_probe_cu_split: tile is a crl_gemm tile code");
  hipError_t e = run_cu_split_probe(gemm_cus, tile, rows, iters, out8);
  if (e == hipErrorInvalidValue) return arg_fail("crl_probe_cu_split: gemm_cus in 8..248 or 256 (no masks), rows a positive multiple of 256, iters >= 1, a tile code crl_gemm accepts for e4m3 operands");
  return e == hipSuccess ? CRL_OK : hip_fail("crl_probe_cu_split", e);
}

}  // extern "C"
