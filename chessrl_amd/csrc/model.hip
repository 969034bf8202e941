// Host-side model runner: owns the packed device weights and the workspace of one
// model and issues the kernel sequence of its forward pass on the caller's stream.
//
// Three architectures share the kernels:
//   GPT64    model_bis.GPT restricted to the 64 board tokens (model_bis.py:358-370):
//            pre-LN blocks, causal attention, logits of token 63 through lm_head.
//   BT4      new_paradigm/value.py BT4: post-LN encoder with relative-position attention,
//            attention-policy head with the dense 4096->1929 map, WDL value head.
//   BT4CLASS the benchmark's BT4-class encoder: post-LN with residual scaling
//            alpha=(2L)^-1/4, mish FFN, generated attention bias (smolgen), attention
//            policy gathered to the 1858-move list, WDL head. Not present in the
//            reference repository; defined by this build.
#include "model.hpp"

#include <cmath>
#include <cstdio>
#include <algorithm>
#include <cstring>

namespace crl {

#define HIPCHK(expr)                                                                      \
  do {                                                                                    \
    hipError_t e_ = (expr);                                                               \
    if (e_ != hipSuccess) {                                                               \
      set_error(std::string(#expr) + ": " + hipGetErrorString(e_));                       \
      return CRL_ERR_HIP;                                                                 \
    }                                                                                     \
  } while (0)

static thread_local std::string g_error;
void set_error(const std::string& s) { g_error = s; }
const char* get_error() { return g_error.c_str(); }

static std::string lkey(const char* fmt, int i) {
  char buf[160];
  std::snprintf(buf, sizeof(buf), fmt, i);
  return buf;
}

Model::Model(const crl_model_config& c) : cfg(c) {
  if (cfg.eps == 0.f) cfg.eps = 1e-5f;
  if (cfg.smolgen_compress == 0) cfg.smolgen_compress = 32;
  if (cfg.smolgen_hidden == 0) cfg.smolgen_hidden = 256;
  if (cfg.smolgen_gen == 0) cfg.smolgen_gen = 256;
  if (cfg.act_dtype != DT_F16) cfg.act_dtype = DT_BF16;
  if (cfg.head_dtype != DT_F16 && cfg.head_dtype != DT_BF16) cfg.head_dtype = cfg.act_dtype;
  if (cfg.micro_batch <= 0) cfg.micro_batch = 4096;
  // tri-state switches: 0 picks the default
  if (cfg.stream_f32 == 0) cfg.stream_f32 = cfg.arch == CRL_ARCH_GPT64 ? 1 : -1;
  if (cfg.ln_fold == 0) cfg.ln_fold = 1;
  if (cfg.fp8_lm_head == 0) cfg.fp8_lm_head = cfg.arch == CRL_ARCH_GPT64 ? 1 : -1;
  cfg.norm_rms = cfg.norm_rms ? 1 : 0;
  vocab = cfg.arch == CRL_ARCH_BT4CLASS ? VOCAB_LEELA : VOCAB_RL;
  const long C = cfg.d_model, F = cfg.d_ff, L = cfg.n_layer, H = cfg.n_head;
  auto add = [&](const std::string& k, long n) { expected.push_back({k, n}); };
  auto lin = [&](const std::string& k, long out, long in, bool bias = true) {
    add(k + ".weight", out * in);
    if (bias) add(k + ".bias", out);
  };
  auto ln = [&](const std::string& k, long n) { add(k + ".weight", n); add(k + ".bias", n); };
  if (cfg.arch == CRL_ARCH_GPT64) {
    lin("FenEncoder.linear1", C, 19); ln("FenEncoder.layernorm1", C);
    add("FenEncoder.ma_gating.a", 64 * C); add("FenEncoder.ma_gating.b", 64 * C);
    for (int i = 0; i < L; ++i) {
      const std::string p = lkey("transformer.h.%d.", i);
      ln(p + "ln_1", C); lin(p + "attn.c_attn", 3 * C, C); lin(p + "attn.c_proj", C, C);
      ln(p + "ln_2", C); lin(p + "mlp.c_fc", F, C); lin(p + "mlp.c_proj", C, F);
    }
    ln("transformer.ln_f", C);
    add("lm_head.weight", (long)VOCAB_RL * C);
    add("pe", 64 * C);
  } else {
    lin("linear1", C, 19); ln("layernorm1", C);
    add("ma_gating.a", 64 * C); add("ma_gating.b", 64 * C);
    for (int i = 0; i < L; ++i) {
      const std::string p = lkey("layers.%d.", i);
      lin(p + "attention.query_proj", C, C); lin(p + "attention.key_proj", C, C);
      lin(p + "attention.value_proj", C, C); lin(p + "attention.out_proj", C, C);
      if (cfg.arch == CRL_ARCH_BT4) {
        add(p + "attention.pos_proj.weight", C * C);
        add(p + "attention.u_bias", C); add(p + "attention.v_bias", C);
      } else {
        const long sc = cfg.smolgen_compress, sh = cfg.smolgen_hidden, sg = cfg.smolgen_gen;
        add(p + "smolgen.compress.weight", sc * C);
        lin(p + "smolgen.hidden", sh, 64 * sc); ln(p + "smolgen.hidden_ln", sh);
        lin(p + "smolgen.gen_from", H * sg, sh); ln(p + "smolgen.gen_from_ln", H * sg);
      }
      ln(p + "norm1", C); ln(p + "norm2", C);
      lin(p + "ff1", F, C); lin(p + "ff2", C, F);
    }
    lin("policy_tokens_lin", C, C); lin("queries_pol", C, C); lin("keys_pol", C, C);
    if (cfg.arch == CRL_ARCH_BT4) add("policy_head.weight", (long)VOCAB_RL * 4096);
    else {
      add("smol_weight_gen.weight", 4096L * cfg.smolgen_gen);
      add("promotion_offsets.weight", 4 * C);
    }
    lin("value_head.dense1", 128, C); lin("value_head.dense2", 128, 128 * 64); lin("value_head.dense3", 3, 128);
  }
  amax_host.assign((size_t)(L + 1) * AMAX_SLOTS, 0.f);
}

Model::~Model() {
  for (void* p : gen_allocs) (void)hipFree(p);
  if (cap_stream) (void)hipStreamDestroy(cap_stream);
  for (void* p : allocs) (void)hipFree(p);
  for (void* p : ws_allocs) (void)hipFree(p);
  for (auto& e : prof_events) { (void)hipEventDestroy(e.a); (void)hipEventDestroy(e.b); }
}

int Model::set_weight(const char* key, const float* data, long numel) {
  if (!key || !data) { set_error("set_weight: null argument"); return CRL_ERR_ARG; }
  std::string k = key;
  if (k == "transformer.wte.weight") return CRL_OK;  // tied to lm_head.weight (model_bis.py:148)
  for (auto& e : expected) {
    if (e.first != k) continue;
    // pe may carry more rows than the 64 board tokens; lm_head may carry padding rows behind the 1929 moves
    // (pretrain_fp8.py:16 trains with vocab_size 1936 so that the fp8 GEMM's N is a multiple of 16).
    const bool grows = k == "pe" || k == "lm_head.weight";
    const bool ok = grows ? (numel >= e.second && numel % cfg.d_model == 0) : numel == e.second;
    if (!ok) { set_error("set_weight: " + k + " has " + std::to_string(numel) + " elements, expected " + std::to_string(e.second)); return CRL_ERR_ARG; }
    // The positional table may carry more rows than the 64 board tokens (block_size rows, model_bis.py:141-146).
    const long keep = grows ? numel : e.second;
    host[k].assign(data, data + keep);
    finalized = false;
    return CRL_OK;
  }
  set_error("set_weight: unexpected key " + k);
  return CRL_ERR_ARG;
}

// ---- device packing ---------------------------------------------------------------------
int Model::dev_alloc(void** p, size_t bytes, bool ws) {
  HIPCHK(hipMalloc(p, bytes ? bytes : 16));
  (ws ? ws_allocs : allocs).push_back(*p);
  return CRL_OK;
}

int Model::upload(const std::vector<float>& v, int dt, float scale, void** out) {
  float* tmp = nullptr;
  HIPCHK(hipMalloc((void**)&tmp, v.size() * sizeof(float)));
  hipError_t e = hipMemcpy(tmp, v.data(), v.size() * sizeof(float), hipMemcpyHostToDevice);
  if (e == hipSuccess) {
    int rc = dev_alloc(out, v.size() * dtype_size(dt), false);
    if (rc) { (void)hipFree(tmp); return rc; }
    e = launch_convert(tmp, *out, (long)v.size(), dt, scale, nullptr);
    if (e == hipSuccess) e = hipDeviceSynchronize();
  }
  (void)hipFree(tmp);
  HIPCHK(e);
  return CRL_OK;
}

const std::vector<float>& Model::w(const std::string& k) { return host.at(k); }

int Model::make_lin(Lin& L, const std::vector<float>& W, const std::vector<float>* bias, int N, int K, int dt16, bool fp8, float amax_all) {
  L.N = N; L.K = K; L.dt = dt16;
  int rc = upload(W, dt16, 1.f, &L.w);
  if (rc) return rc;
  if (fp8) {
    float am = amax_all > 0.f ? amax_all : 0.f;
    for (float x : W) am = std::fmax(am, std::fabs(x));
    L.wscale = am > 0.f ? 448.f / am : 1.f;
    rc = upload(W, DT_FP8, L.wscale, &L.w8);
    if (rc) return rc;
  }
  if (bias) {
    rc = upload(*bias, DT_F32, 1.f, (void**)&L.b);
    if (rc) return rc;
  }
  return CRL_OK;
}

static std::vector<float> cat(std::initializer_list<const std::vector<float>*> parts) {
  std::vector<float> r;
  for (auto* p : parts) r.insert(r.end(), p->begin(), p->end());
  return r;
}

int Model::finalize() {
  for (auto& e : expected)
    if (!host.count(e.first)) { set_error("finalize: missing weight " + e.first); return CRL_ERR_STATE; }
  for (void* p : allocs) (void)hipFree(p);
  allocs.clear();
  layers.assign(cfg.n_layer, Layer());
  const int C = cfg.d_model, F = cfg.d_ff, H = cfg.n_head;
  const bool f8 = cfg.fp8 != 0;
  const int hd = cfg.head_dtype, ad = cfg.act_dtype;
  int rc;
#define UP(vec, dt, out) do { rc = upload(vec, dt, 1.f, (void**)&(out)); if (rc) return rc; } while (0)
#define LIN(L, W, B, N, K, dt, f) do { rc = make_lin(L, W, B, N, K, dt, f); if (rc) return rc; } while (0)
  const std::string pre = cfg.arch == CRL_ARCH_GPT64 ? "FenEncoder." : "";
  {
    const auto& w1 = w(pre + "linear1.weight");  // [C,19] -> [19,C]
    std::vector<float> w1t((size_t)19 * C);
    for (int c = 0; c < C; ++c)
      for (int p = 0; p < 19; ++p) w1t[(size_t)p * C + c] = w1[(size_t)c * 19 + p];
    UP(w1t, DT_F32, emb_w1t);
    UP(w(pre + "linear1.bias"), DT_F32, emb_b1);
    UP(w(pre + "layernorm1.weight"), DT_F32, emb_g);
    UP(w(pre + "layernorm1.bias"), DT_F32, emb_b);
    std::vector<float> ea = w(pre + "ma_gating.a");
    for (float& x : ea) x = std::exp(x);
    UP(ea, DT_F32, gate_a_exp);
    UP(w(pre + "ma_gating.b"), DT_F32, gate_b);
  }
  if (cfg.arch == CRL_ARCH_GPT64) {
    UP(w("pe"), DT_F32, pe_f32);
    pe_rows = (int)(w("pe").size() / (size_t)C);
    // The first 1929 rows of lm_head are the moves; a checkpoint trained with a padded vocabulary has more. The e4m3
    // scale is per tensor, so it is taken over every row the checkpoint holds.
    std::vector<float> head_w(w("lm_head.weight").begin(), w("lm_head.weight").begin() + (size_t)VOCAB_RL * C);
    float head_amax = 0.f;
    for (float x : w("lm_head.weight")) head_amax = std::fmax(head_amax, std::fabs(x));
    UP(head_w, DT_F32, wte_f32);   // token embedding, tied to the output head (model_bis.py:148)
    for (int i = 0; i < cfg.n_layer; ++i) {
      Layer& ly = layers[i];
      const std::string p = lkey("transformer.h.%d.", i);
      UP(w(p + "ln_1.weight"), DT_F32, ly.ln1_g); UP(w(p + "ln_1.bias"), DT_F32, ly.ln1_b);
      UP(w(p + "ln_2.weight"), DT_F32, ly.ln2_g); UP(w(p + "ln_2.bias"), DT_F32, ly.ln2_b);
      LIN(ly.qkv, w(p + "attn.c_attn.weight"), &w(p + "attn.c_attn.bias"), 3 * C, C, ad, f8);
      LIN(ly.proj, w(p + "attn.c_proj.weight"), &w(p + "attn.c_proj.bias"), C, C, ad, f8);
      LIN(ly.ff1, w(p + "mlp.c_fc.weight"), &w(p + "mlp.c_fc.bias"), F, C, ad, f8);
      LIN(ly.ff2, w(p + "mlp.c_proj.weight"), &w(p + "mlp.c_proj.bias"), C, F, ad, f8);
    }
    UP(w("transformer.ln_f.weight"), DT_F32, lnf_g); UP(w("transformer.ln_f.bias"), DT_F32, lnf_b);
    rc = make_lin(lm_head, head_w, nullptr, VOCAB_RL, C, hd, f8 && cfg.fp8_lm_head > 0, head_amax); if (rc) return rc;
  } else {
    // Absolute sinusoid table of new_paradigm/value.py:77-93.
    std::vector<float> pe((size_t)64 * C);
    for (int p = 0; p < 64; ++p)
      for (int i = 0; i < C; i += 2) {
        const float d = std::pow(10000.0f, (float)i / (float)C);
        pe[(size_t)p * C + i] = std::sin((float)p / d);
        if (i + 1 < C) pe[(size_t)p * C + i + 1] = std::cos((float)p / d);
      }
    UP(pe, hd, pe_head);
    for (int i = 0; i < cfg.n_layer; ++i) {
      Layer& ly = layers[i];
      const std::string p = lkey("layers.%d.", i);
      std::vector<float> wq = cat({&w(p + "attention.query_proj.weight"), &w(p + "attention.key_proj.weight"), &w(p + "attention.value_proj.weight")});
      std::vector<float> bq = cat({&w(p + "attention.query_proj.bias"), &w(p + "attention.key_proj.bias"), &w(p + "attention.value_proj.bias")});
      int nq = 3 * C;
      if (qk_paired()) {
        // Output columns [q_0 | k_0 | q_1 | k_1 | ...] then v: a head's q and k of one token are one whole 128-byte line.
        const int hsz = C / cfg.n_head;
        std::vector<float> wp(wq), bp(bq);
        for (int h = 0; h < cfg.n_head; ++h)
          for (int part = 0; part < 2; ++part)
            for (int r = 0; r < hsz; ++r) {
              const size_t src = (size_t)part * C + (size_t)h * hsz + r, dst = ((size_t)h * 2 + part) * hsz + r;
              std::copy(wq.begin() + src * C, wq.begin() + (src + 1) * C, wp.begin() + dst * C);
              bp[dst] = bq[src];
            }
        wq.swap(wp); bq.swap(bp);
      }
      if (cfg.arch == CRL_ARCH_BT4CLASS) {
        const auto& cw = w(p + "smolgen.compress.weight");
        wq.insert(wq.end(), cw.begin(), cw.end());
        bq.insert(bq.end(), (size_t)cfg.smolgen_compress, 0.f);
        nq += cfg.smolgen_compress;
      }
      LIN(ly.qkv, wq, &bq, nq, C, ad, f8);
      LIN(ly.proj, w(p + "attention.out_proj.weight"), &w(p + "attention.out_proj.bias"), C, C, ad, f8);
      LIN(ly.ff1, w(p + "ff1.weight"), &w(p + "ff1.bias"), F, C, ad, f8);
      LIN(ly.ff2, w(p + "ff2.weight"), &w(p + "ff2.bias"), C, F, ad, f8);
      UP(w(p + "norm1.weight"), DT_F32, ly.ln1_g); UP(w(p + "norm1.bias"), DT_F32, ly.ln1_b);
      UP(w(p + "norm2.weight"), DT_F32, ly.ln2_g); UP(w(p + "norm2.bias"), DT_F32, ly.ln2_b);
      if (cfg.arch == CRL_ARCH_BT4) {
        // pos_proj(PE) does not depend on the input (new_paradigm/attn.py:505): fold it here.
        const auto& pw = w(p + "attention.pos_proj.weight");
        std::vector<float> pt((size_t)64 * C);
        for (int t = 0; t < 64; ++t)
          for (int o = 0; o < C; ++o) {
            double s = 0;
            for (int c = 0; c < C; ++c) s += (double)pe[(size_t)t * C + c] * pw[(size_t)o * C + c];
            pt[(size_t)t * C + o] = (float)s;
          }
        UP(pt, ad, ly.pos);
        UP(w(p + "attention.u_bias"), DT_F32, ly.u_bias);
        UP(w(p + "attention.v_bias"), DT_F32, ly.v_bias);
      } else {
        const int sc = cfg.smolgen_compress, sh = cfg.smolgen_hidden, sg = cfg.smolgen_gen;
        LIN(ly.sm_hidden, w(p + "smolgen.hidden.weight"), &w(p + "smolgen.hidden.bias"), sh, 64 * sc, ad, false);
        LIN(ly.sm_gen, w(p + "smolgen.gen_from.weight"), &w(p + "smolgen.gen_from.bias"), H * sg, sh, ad, false);
        UP(w(p + "smolgen.hidden_ln.weight"), DT_F32, ly.sm_ln1_g); UP(w(p + "smolgen.hidden_ln.bias"), DT_F32, ly.sm_ln1_b);
        UP(w(p + "smolgen.gen_from_ln.weight"), DT_F32, ly.sm_ln2_g); UP(w(p + "smolgen.gen_from_ln.bias"), DT_F32, ly.sm_ln2_b);
      }
    }
    // The reference's fp8 recipe turns every nn.Linear of the model into a te.Linear, the output head included
    // (model_fp8.py:43,45,90,92,140): in the e4m3 BT4-class model the three head linears that run on every token
    // (policy_tokens_lin, queries_pol|keys_pol, value_head.dense1) get e4m3 copies too. dense2 and dense3 (one row per
    // position) stay 16-bit. Off unless asked for (cfg.fp8_lm_head = 1): on the benchmark model it takes 0.8 ms off a
    // 49 ms pass and adds half again to the policy error against fp32.
    const bool f8heads = f8 && cfg.arch == CRL_ARCH_BT4CLASS && cfg.fp8_lm_head > 0;
    LIN(pol_tok, w("policy_tokens_lin.weight"), &w("policy_tokens_lin.bias"), C, C, hd, f8heads);
    {
      std::vector<float> wqk = cat({&w("queries_pol.weight"), &w("keys_pol.weight")});
      std::vector<float> bqk = cat({&w("queries_pol.bias"), &w("keys_pol.bias")});
      LIN(pol_qk, wqk, &bqk, 2 * C, C, hd, f8heads);
    }
    if (cfg.arch == CRL_ARCH_BT4) {
      LIN(pol_head, w("policy_head.weight"), nullptr, VOCAB_RL, 4096, hd, false);
    } else {
      // Rows of the shared bias generator are stored in the order the attention kernel
      // reads its accumulator registers, so the generated tile needs no transpose.
      const int sg = cfg.smolgen_gen;
      const auto& gw = w("smol_weight_gen.weight");
      std::vector<float> perm((size_t)4096 * sg);
      for (int i = 0; i < 64; ++i)
        for (int j = 0; j < 64; ++j)
          std::memcpy(&perm[(size_t)attn_bias_slot_host(i, j) * sg], &gw[(size_t)(i * 64 + j) * sg], sizeof(float) * sg);
      LIN(sm_weight_gen, perm, nullptr, 4096, sg, ad, f8);
      UP(w("promotion_offsets.weight"), DT_F32, promo_w);
      // Gather tables: Leela move v -> (from_token*64+to_token) for black / white rows.
      std::vector<int16_t> gi((size_t)2 * VOCAB_LEELA);
      std::vector<int8_t> gp(VOCAB_LEELA);
      const auto& names = policy_leela();
      for (int v = 0; v < VOCAB_LEELA; ++v) {
        const std::string& s = names[v];
        const int ff = s[0] - 'a', fr = s[1] - '1', tf = s[2] - 'a', tr = s[3] - '1';
        // white row: squares as written; black row: ranks mirrored back to the real board.
        gi[VOCAB_LEELA + v] = (int16_t)(((7 - fr) * 8 + ff) * 64 + ((7 - tr) * 8 + tf));
        gi[v] = (int16_t)((fr * 8 + ff) * 64 + (tr * 8 + tf));
        gp[v] = s.size() == 5 ? (int8_t)(tf * 4 + (s[4] == 'q' ? 0 : s[4] == 'r' ? 1 : 2)) : (int8_t)-1;
      }
      rc = dev_alloc((void**)&gidx, gi.size() * 2, false); if (rc) return rc;
      rc = dev_alloc((void**)&gpromo, gp.size(), false); if (rc) return rc;
      HIPCHK(hipMemcpy(gidx, gi.data(), gi.size() * 2, hipMemcpyHostToDevice));
      HIPCHK(hipMemcpy(gpromo, gp.data(), gp.size(), hipMemcpyHostToDevice));
    }
    LIN(val1, w("value_head.dense1.weight"), &w("value_head.dense1.bias"), 128, C, hd, f8heads);
    LIN(val2, w("value_head.dense2.weight"), &w("value_head.dense2.bias"), 128, 8192, hd, false);
    LIN(val3, w("value_head.dense3.weight"), &w("value_head.dense3.bias"), 3, 128, hd, false);
  }
  rc = dev_alloc((void**)&amax_dev, sizeof(float) * amax_host.size(), false);
  if (rc) return rc;
  HIPCHK(hipMemset(amax_dev, 0, sizeof(float) * amax_host.size()));
#undef UP
#undef LIN
  finalized = true;
  return CRL_OK;
}

// ---- workspace ------------------------------------------------------------------------------
int Model::ensure_ws(int mb) {
  if (mb <= ws_mb) return CRL_OK;
  for (void* p : ws_allocs) (void)hipFree(p);
  ws_allocs.clear();
  ws_mb = 0;
  const size_t M = (size_t)mb * 64, C = cfg.d_model, F = cfg.d_ff, H = cfg.n_head;
  int rc;
#define WS(ptr, bytes) do { rc = dev_alloc((void**)&(ptr), (bytes), true); if (rc) return rc; } while (0)
  const bool sf32_post = cfg.arch != CRL_ARCH_GPT64 && cfg.stream_f32 > 0;   // post-LN trunks keep x, t and h in the stream's type
  WS(ws.x, M * C * 4);        // residual stream (fp32 with stream_f32, else 16-bit)
  WS(ws.x8, M * C);
  WS(ws.t, M * C * (sf32_post ? 4 : 2));
  WS(ws.h, M * C * (sf32_post ? 4 : 2));
  WS(ws.h8, M * C);
  if (sf32_post) { WS(ws.x16, M * C * 2); WS(ws.h16, M * C * 2); }
  WS(ws.qkv, M * 3 * C * 2);
  WS(ws.ao, M * C * 2);
  WS(ws.ao8, M * C);
  WS(ws.f, M * F * 2);
  WS(ws.f8, M * F);
  WS(ws.stm, (size_t)mb);
  WS(ws.st1, M * 2 * sizeof(float));
  WS(ws.st2, M * 2 * sizeof(float));
  WS(ws.splitk, (size_t)Workspace::SPLITK_BYTES);
  if (cfg.arch == CRL_ARCH_BT4CLASS) {
    WS(ws.comp, M * cfg.smolgen_compress * 2);
    WS(ws.sh1, (size_t)mb * cfg.smolgen_hidden * 2);
    WS(ws.sh2, (size_t)mb * cfg.smolgen_hidden * 2);
    WS(ws.sg1, (size_t)mb * H * cfg.smolgen_gen * 2);
    WS(ws.sg2, (size_t)mb * H * cfg.smolgen_gen * 2);
    WS(ws.sg2_8, (size_t)mb * H * cfg.smolgen_gen);
    WS(ws.bias, (size_t)mb * H * 4096 * 2);
  }
  if (cfg.arch == CRL_ARCH_GPT64) {
    WS(ws.hl, (size_t)mb * C * 2);
    WS(ws.hl8, (size_t)mb * C);
  } else {
    WS(ws.tok, M * C * 2);
    WS(ws.pqk, M * 2 * C * 2);
    WS(ws.v1, M * 128 * 2);
    WS(ws.v2, (size_t)mb * 128 * 2);
    WS(ws.dense, (size_t)mb * 4096 * 2);
  }
#undef WS
  ws_mb = mb;
  return CRL_OK;
}

// ---- profiling helpers ------------------------------------------------------------------------
void Model::prof_begin(int fam, hipStream_t st) {
  if (!profiling) return;
  if (prof_used == prof_events.size()) {
    ProfEvent e;
    (void)hipEventCreate(&e.a);
    (void)hipEventCreate(&e.b);
    prof_events.push_back(e);
  }
  prof_events[prof_used].fam = fam;
  (void)hipEventRecord(prof_events[prof_used].a, st);
}
void Model::prof_end(hipStream_t st) {
  if (!profiling) return;
  (void)hipEventRecord(prof_events[prof_used].b, st);
  ++prof_used;
}
void Model::prof_collect(hipStream_t st) {
  if (!profiling) return;
  (void)hipStreamSynchronize(st);
  for (size_t i = 0; i < prof_used; ++i) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, prof_events[i].a, prof_events[i].b) == hipSuccess) {
      prof_ms[prof_events[i].fam] += ms;
      prof_n[prof_events[i].fam] += 1;
    }
  }
  prof_used = 0;
}

// ---- launch helpers ------------------------------------------------------------------------------
struct GOpt {
  int act = ACT_NONE;
  float alpha = 1.f;
  const void* res = nullptr; long ldr = 0; int res_dt = DT_BF16; int res_rows = 0;
  float a_scale = 1.f;     // scale the fp8 A operand was quantised with
  float out_scale = 1.f;
  float* amax = nullptr;
  void* C2 = nullptr; long ldc2 = 0; int nsplit = 0;
  bool k_parallel = false;  // token steps of generation: few rows, so K is spread over more waves (different summation order)
  // LayerNorm that follows this GEMM, to be folded into it where the GEMM kernel can (*ln_folded says whether it did).
  const float* ln_g = nullptr; const float* ln_b = nullptr; void* ln_out = nullptr; int ln_dt = DT_BF16; bool* ln_folded = nullptr;
  // The residual is LayerNorm(res), normalised in the epilogue from these row statistics, gain and offset.
  const float* res_stats = nullptr; const float* res_g = nullptr; const float* res_b = nullptr;
  // Ask for the blocked output layout (GemmArgs::c_blocked) where the GEMM has a kernel for it; *c_blocked says whether it was used.
  bool* c_blocked = nullptr;
};

int Model::gemm(const Lin& L, const void* A, long lda, int in_dt, void* C, long ldc, int out_dt, int M, const GOpt& o, hipStream_t st) {
  GemmArgs g;
  std::memset(&g, 0, sizeof(g));
  g.A = A; g.lda = lda;
  g.W = in_dt == DT_FP8 ? L.w8 : L.w; g.ldw = L.K;
  if (!g.W) { set_error("gemm: weight copy for the requested element type is missing"); return CRL_ERR_STATE; }
  g.C = C; g.ldc = ldc; g.C2 = o.C2; g.ldc2 = o.ldc2; g.nsplit = o.nsplit > 0 ? o.nsplit : L.N;
  g.bias = L.b; g.res = o.res; g.ldr = o.ldr; g.res_dtype = o.res_dt; g.res_rows = o.res_rows;
  g.amax = o.amax; g.M = M; g.N = L.N; g.K = L.K; g.act = o.act;
  g.res_stats = o.res_stats; g.res_gamma = o.res_g; g.res_beta = cfg.norm_rms ? nullptr : o.res_b;
  g.descale = in_dt == DT_FP8 ? 1.f / (o.a_scale * L.wscale) : 1.f;
  g.alpha = o.alpha; g.out_scale = o.out_scale;
  // Few rows: K spread over more waves (another summation order; the token steps of generation always, the forward pass
  // only where the model was told that a position's bits may depend on the batch it travels in).
  g.k_parallel = o.k_parallel ? 1 : 0;
  g.splitk_ws = ws.splitk; g.splitk_ws_bytes = Workspace::SPLITK_BYTES;
  if (o.ln_out) {
    g.nsplit = g.N;
    g.ln_gamma = o.ln_g; g.ln_beta = o.ln_b; g.ln_out = o.ln_out; g.ln_ldo = L.N; g.ln_out_dtype = o.ln_dt; g.ln_eps = cfg.eps;
    g.ln_rms = cfg.norm_rms;
    const bool fold = !profiling && gemm_folds_layernorm(g, in_dt == DT_FP8 ? DT_FP8 : L.dt);
    if (o.ln_folded) *o.ln_folded = fold;
    if (!fold) { g.ln_gamma = g.ln_beta = nullptr; g.ln_out = nullptr; }
  }
  if (o.c_blocked) {
    g.c_blocked = 1;
    if (!gemm_shortk_can(g, in_dt == DT_FP8 ? DT_FP8 : L.dt, out_dt)) g.c_blocked = 0;
    *o.c_blocked = g.c_blocked != 0;
  }
  const int fam = in_dt == DT_FP8 ? 0 : 5;
  if (profiling) prof_flops[fam] += 2.0 * M * (double)L.N * L.K;
  prof_begin(fam, st);
  hipError_t e = launch_gemm(g, in_dt == DT_FP8 ? DT_FP8 : L.dt, out_dt, 0, st);
  prof_end(st);
  HIPCHK(e);
  return CRL_OK;
}

// trunk: one of the norms cfg.norm_rms turns into RMSNorm (the stem's and the bias generator's stay LayerNorm).
int Model::lnorm(const void* x, long ldx, int in_dt, const float* g, const float* b, void* out, int out_dt, uint8_t* out8,
                 float scale8, long ldo, int rows, int C, float* amax, hipStream_t st, float* stats, void* out_b, int out_b_dt, bool trunk) {
  LayerNormArgs a;
  std::memset(&a, 0, sizeof(a));
  a.x = x; a.ldx = ldx; a.in_dtype = in_dt; a.gamma = g; a.beta = b; a.out = out; a.out_dtype = out_dt;
  a.out_fp8 = out8; a.fp8_scale = scale8; a.ldo = ldo; a.rows = rows; a.C = C; a.eps = cfg.eps; a.amax = amax; a.stats = stats;
  a.out_b = out_b; a.out_b_dtype = out_b_dt; a.rms = (trunk && cfg.norm_rms) ? 1 : 0;
  prof_begin(2, st);
  hipError_t e = launch_layernorm(a, st);
  prof_end(st);
  HIPCHK(e);
  return CRL_OK;
}

float Model::act_scale(int layer, int slot) const {
  const float am = amax_host[(size_t)layer * AMAX_SLOTS + slot];
  return am > 0.f ? 448.f / am : 1.f;
}

int Model::forward(const float* planes, const uint8_t* ids, const uint8_t* flags, int B, float* policy, float* wdl,
                   bool calibrate, hipStream_t st) {
  if (!policy) { set_error("forward: bad arguments"); return CRL_ERR_ARG; }
  return forward_tokens(planes, ids, flags, nullptr, 0, B, policy, nullptr, wdl, calibrate, st);
}

int Model::forward_tokens(const float* planes, const uint8_t* ids, const uint8_t* flags, const int64_t* idx, int t, int B,
                          float* policy, float* all_logits, float* wdl, bool calibrate, hipStream_t st) {
  if (!finalized) { set_error("forward: call crl_model_finalize first"); return CRL_ERR_STATE; }
  if (B < 0 || t < 0 || (!planes && !(ids && flags)) || (!policy && !all_logits)) { set_error("forward: bad arguments"); return CRL_ERR_ARG; }
  if ((t > 0 || all_logits) && cfg.arch != CRL_ARCH_GPT64) { set_error("forward: move tokens and per-token logits exist only for CRL_ARCH_GPT64"); return CRL_ERR_ARG; }
  if (t > 0 && !idx) { set_error("forward: move tokens missing"); return CRL_ERR_ARG; }
  const int T = 64 + t;
  if (t > 0 && T > pe_rows) { set_error("forward: " + std::to_string(T) + " tokens exceed the " + std::to_string(pe_rows) + " rows of the positional table"); return CRL_ERR_ARG; }
  // The workspace is counted in 64-token units; longer positions take proportionally fewer per micro-batch.
  const int mbmax = std::max(1, (int)((long)cfg.micro_batch * 64 / T));
  const int mb0 = B < mbmax ? B : mbmax;
  int rc = ensure_ws((int)(((long)mb0 * T + 63) / 64));
  if (rc) return rc;
  for (int b0 = 0; b0 < B; b0 += mbmax) {
    const int mb = (B - b0) < mbmax ? (B - b0) : mbmax;
    rc = forward_chunk(planes ? planes + (size_t)b0 * 64 * 19 : nullptr, ids ? ids + (size_t)b0 * 64 : nullptr,
                       flags ? flags + (size_t)b0 * 4 : nullptr, idx ? idx + (size_t)b0 * t : nullptr, t, mb,
                       policy ? policy + (size_t)b0 * vocab : nullptr, all_logits ? all_logits + (size_t)b0 * T * vocab : nullptr,
                       wdl ? wdl + (size_t)b0 * 3 : nullptr, calibrate, st);
    if (rc) return rc;
  }
  prof_collect(st);
  return CRL_OK;
}

int Model::forward_chunk(const float* planes, const uint8_t* ids, const uint8_t* flags, const int64_t* idx, int t, int mb,
                         float* policy, float* all_logits, float* wdl, bool calibrate, hipStream_t st, const LayerWindow* win) {
  const int C = cfg.d_model, F = cfg.d_ff, H = cfg.n_head, L = cfg.n_layer, hs = C / H;
  // Layers [l0, l1) of this call: the whole trunk, or the window of run_layers (its input comes from the caller instead of
  // the embedding, its first layer reads that input as a plain residual and its last one writes the 16-bit output).
  const int l0 = win ? win->first : 0, l1 = win ? win->last : L;
  const int T = 64 + t;          // tokens per position: the board, then t move tokens (CRL_ARCH_GPT64 only)
  const int M = mb * T;
  const bool f8 = cfg.fp8 && !calibrate && !force_16bit;
  const int hd = cfg.head_dtype, ad = cfg.act_dtype;
  const bool gpt = cfg.arch == CRL_ARCH_GPT64;
  // fp32 residual stream: GPT64 keeps x in fp32; the post-LN trunks keep x, t and h in fp32 and hand the products a
  // 16-bit (or e4m3) operand copy written by the same LayerNorm launch.
  const bool sf32 = cfg.stream_f32 > 0 && (gpt || L > 0);
  const bool sf32p = sf32 && !gpt;
  const int xdt = sf32 ? DT_F32 : ad;
  auto am = [&](int l, int slot) -> float* { return calibrate ? amax_dev + (size_t)l * AMAX_SLOTS + slot : nullptr; };
  int rc;
#define RUN(call) do { rc = (call); if (rc) return rc; } while (0)

  // ---- embedding
  if (win) {
    const long n = (long)M * C;
    HIPCHK(launch_convert(win->x_in, ws.x, n, xdt, 1.f, st));
    if (f8 && !gpt) HIPCHK(launch_convert(win->x_in, ws.x8, n, DT_FP8, act_scale(l0, 0), st));
    if (sf32p && !f8) HIPCHK(launch_convert(win->x_in, ws.x16, n, ad, 1.f, st));
  } else {
    EmbedArgs e;
    std::memset(&e, 0, sizeof(e));
    e.planes = planes; e.ids = ids; e.flags = flags;
    e.w1t = emb_w1t; e.b1 = emb_b1; e.ln_g = emb_g; e.ln_b = emb_b; e.gate_a_exp = gate_a_exp; e.gate_b = gate_b;
    e.pe = gpt ? pe_f32 : nullptr;
    e.out = ws.x; e.out_dtype = (L == 0 && !gpt) ? hd : xdt; e.tokens = mb * 64; e.C = C; e.act = ACT_GELU; e.eps = cfg.eps;
    e.out_T = T;
    if (!gpt && L > 0) { e.out_fp8 = f8 ? ws.x8 : nullptr; e.fp8_scale = f8 ? act_scale(0, 0) : 1.f; e.amax = am(0, 0); }
    if (sf32p && !f8) { e.out_b = ws.x16; e.out_b_dtype = ad; }
    prof_begin(3, st);
    hipError_t he = launch_embed(e, st);
    prof_end(st);
    HIPCHK(he);
    if (t > 0) {
      TokenEmbedArgs te;
      std::memset(&te, 0, sizeof(te));
      te.idx = idx; te.wte = wte_f32; te.pe = pe_f32; te.out = ws.x; te.B = mb; te.t = t; te.T = T; te.C = C; te.V = VOCAB_RL; te.out_dtype = xdt;
      prof_begin(3, st);
      he = launch_token_embed(te, st);
      prof_end(st);
      HIPCHK(he);
    }
  }
  if (cfg.arch == CRL_ARCH_BT4CLASS && !win) {
    HIPCHK(launch_extract_stm(planes, flags, ws.stm, mb, st));
  }

  // BT4-class in e4m3 with bf16 activations: the normalised activations are not written in 16 bits at all (every
  // tile size has the residual-normalising epilogue, so this does not depend on the batch).
  const bool fold = cfg.ln_fold > 0 && f8 && cfg.arch == CRL_ARCH_BT4CLASS && ad == DT_BF16 && !sf32;
  // e4m3 head linears (BT4-class): the trunk's last norm writes the e4m3 copy the policy-token and value linears read
  // (scale from the first entry of the amax table's last row), the policy-token linear writes its output in e4m3 for
  // the query|key linear (second entry). Rows that were never calibrated keep the heads on their 16-bit copies.
  const bool f8h = f8 && !win && cfg.arch == CRL_ARCH_BT4CLASS && L > 0 && pol_tok.w8 != nullptr && amax_host[(size_t)L * AMAX_SLOTS] > 0.f &&
                   amax_host[(size_t)L * AMAX_SLOTS + 1] > 0.f;
  const bool cal_heads = calibrate && cfg.arch == CRL_ARCH_BT4CLASS && L > 0;
  // 16-bit operand copies of x and h (the tensors themselves when the stream is 16-bit)
  void* const x_op = sf32p ? ws.x16 : ws.x;
  void* const h_op = sf32p ? ws.h16 : ws.h;
  const float attn_scale = cfg.arch == CRL_ARCH_BT4 ? 1.0f / std::sqrt((float)C) : 1.0f / std::sqrt((float)hs);
  const float alpha = cfg.arch == CRL_ARCH_BT4CLASS ? std::pow(2.0f * (float)L, -0.25f) : 1.0f;

  for (int l = l0; l < l1; ++l) {
    const Layer& ly = layers[l];
    const bool last = l + 1 == l1;
    const void* a_in; int a_dt; float a_sc = 1.f;
    if (gpt) {
      // h = LN1(x)
      RUN(lnorm(ws.x, C, xdt, ly.ln1_g, ly.ln1_b, f8 ? nullptr : ws.h, ad, f8 ? ws.h8 : nullptr, f8 ? act_scale(l, 0) : 1.f, C, M, C, am(l, 0), st));
      a_in = f8 ? (const void*)ws.h8 : (const void*)ws.h; a_dt = f8 ? DT_FP8 : ad; a_sc = f8 ? act_scale(l, 0) : 1.f;
    } else {
      a_in = f8 ? (const void*)ws.x8 : (const void*)x_op; a_dt = f8 ? DT_FP8 : ad; a_sc = f8 ? act_scale(l, 0) : 1.f;
    }
    // q|k|v (and the smolgen compression for BT4-class) in one GEMM
    {
      GOpt o; o.a_scale = a_sc;
      if (cfg.arch == CRL_ARCH_BT4CLASS) { o.C2 = ws.comp; o.ldc2 = cfg.smolgen_compress; o.nsplit = 3 * C; }
      RUN(gemm(ly.qkv, a_in, C, a_dt, ws.qkv, 3 * C, ad, M, o, st));
    }
    if (kv_capture) HIPCHK(launch_kv_store(ws.qkv, kv_layers[l], mb, T, kv_Tmax, C, st));
    const void* bias_tile = nullptr;
    bool bias_blocked = false;
    if (cfg.arch == CRL_ARCH_BT4CLASS) {
      const int sc = cfg.smolgen_compress, sh = cfg.smolgen_hidden, sg = cfg.smolgen_gen;
      GOpt o; o.act = ACT_SWISH;
      RUN(gemm(ly.sm_hidden, ws.comp, 64 * sc, ad, ws.sh1, sh, ad, mb, o, st));
      RUN(lnorm(ws.sh1, sh, ad, ly.sm_ln1_g, ly.sm_ln1_b, ws.sh2, ad, nullptr, 1.f, sh, mb, sh, nullptr, st, nullptr, nullptr, DT_BF16, false));
      RUN(gemm(ly.sm_gen, ws.sh2, sh, ad, ws.sg1, H * sg, ad, mb, o, st));
      // The shared 256 -> 4096 generator is the largest smolgen product (2*B*H*256*4096 per layer): in the fp8
      // configuration it takes e4m3 inputs like the trunk linears; the two small layers before it stay 16-bit.
      RUN(lnorm(ws.sg1, H * sg, ad, ly.sm_ln2_g, ly.sm_ln2_b, f8 ? nullptr : ws.sg2, ad, f8 ? ws.sg2_8 : nullptr, f8 ? act_scale(l, 4) : 1.f,
                H * sg, mb, H * sg, am(l, 4), st, nullptr, nullptr, DT_BF16, false));
      // (with e4m3 inputs and whole blocks of 256 (position, head) rows the product is written in the blocked layout,
      // which the attention kernel reads as it stands)
      GOpt o2; o2.a_scale = f8 ? act_scale(l, 4) : 1.f; o2.c_blocked = &bias_blocked;
      RUN(gemm(sm_weight_gen, f8 ? (const void*)ws.sg2_8 : (const void*)ws.sg2, sg, f8 ? DT_FP8 : ad, ws.bias, 4096, ad, mb * H, o2, st));
      bias_tile = ws.bias;
    }
    // attention
    {
      AttnArgs a;
      std::memset(&a, 0, sizeof(a));
      const uint16_t* base = reinterpret_cast<const uint16_t*>(ws.qkv);
      if (!gpt && qk_paired()) { a.q = base; a.k = base + hs; a.qk_hstride = 2 * hs; }
      else { a.q = base; a.k = base + C; }
      a.v = base + 2 * C; a.ldq = a.ldk = a.ldv = 3 * C;
      a.bias = bias_tile; a.bias_blocked = bias_blocked ? 1 : 0; a.pos = ly.pos; a.u_bias = ly.u_bias; a.v_bias = ly.v_bias;
      a.out = f8 ? (void*)ws.ao8 : (void*)ws.ao; a.ldo = C; a.out_dtype = f8 ? DT_FP8 : ad;
      a.out_scale = f8 ? act_scale(l, 1) : 1.f; a.amax = am(l, 1);
      a.B = mb; a.H = H; a.scale = attn_scale; a.in_dtype = ad; a.T = T;
      a.mode = gpt ? ATTN_CAUSAL : cfg.arch == CRL_ARCH_BT4 ? ATTN_RELSHIFT : ATTN_BIAS;
      prof_begin(1, st);
      hipError_t he = launch_attention(a, hs, st);
      prof_end(st);
      HIPCHK(he);
    }
    const void* ao_in = f8 ? (const void*)ws.ao8 : (const void*)ws.ao;
    const int ao_dt = f8 ? DT_FP8 : ad;
    if (gpt) {
      // x += proj(ao);  h = LN2(x);  x += proj2(gelu(fc(h)))
      { GOpt o; o.res = ws.x; o.ldr = C; o.res_dt = xdt; o.a_scale = f8 ? act_scale(l, 1) : 1.f;
        RUN(gemm(ly.proj, ao_in, C, ao_dt, ws.x, C, xdt, M, o, st)); }
      RUN(lnorm(ws.x, C, xdt, ly.ln2_g, ly.ln2_b, f8 ? nullptr : ws.h, ad, f8 ? ws.h8 : nullptr, f8 ? act_scale(l, 2) : 1.f, C, M, C, am(l, 2), st));
      { GOpt o; o.act = ACT_GELU; o.a_scale = f8 ? act_scale(l, 2) : 1.f; o.out_scale = f8 ? act_scale(l, 3) : 1.f; o.amax = am(l, 3);
        RUN(gemm(ly.ff1, f8 ? (const void*)ws.h8 : (const void*)ws.h, C, ao_dt, f8 ? (void*)ws.f8 : (void*)ws.f, F, ao_dt, M, o, st)); }
      { GOpt o; o.res = ws.x; o.ldr = C; o.res_dt = xdt; o.a_scale = f8 ? act_scale(l, 3) : 1.f;
        RUN(gemm(ly.ff2, f8 ? (const void*)ws.f8 : (const void*)ws.f, F, ao_dt, ws.x, C, xdt, M, o, st)); }
    } else {
      // t = x + alpha*proj(ao);  h = LN1(t). With `fold` the normalised tensors x and h exist only as e4m3 copies
      // (the products' operands): the LayerNorm launches leave their row statistics behind, and the product that
      // takes x or h as its residual re-normalises the un-normalised tensor t in its epilogue, writing in place.
      // With an fp32 stream x, t and h are fp32 and every norm also writes the 16-bit operand copy (x16, h16).
      { GOpt o; o.res = ws.x; o.ldr = C; o.res_dt = xdt; o.alpha = alpha; o.a_scale = f8 ? act_scale(l, 1) : 1.f;
        if (fold && l > l0) { o.res = ws.t; o.res_stats = ws.st2; o.res_g = layers[l - 1].ln2_g; o.res_b = layers[l - 1].ln2_b; }
        RUN(gemm(ly.proj, ao_in, C, ao_dt, ws.t, C, xdt, M, o, st)); }
      RUN(lnorm(ws.t, C, xdt, ly.ln1_g, ly.ln1_b, fold ? nullptr : ws.h, xdt, f8 ? ws.h8 : nullptr, f8 ? act_scale(l, 2) : 1.f, C, M, C, am(l, 2), st,
                fold ? ws.st1 : nullptr, (sf32p && !f8) ? ws.h16 : nullptr, ad));
      const void* h_in = f8 ? (const void*)ws.h8 : (const void*)h_op;
      if (cfg.arch == CRL_ARCH_BT4) {
        // y = ff2(ff1(h)) with no activation in between; t = gelu(y) + h (new_paradigm/value.py:65-70)
        { GOpt o; o.a_scale = f8 ? act_scale(l, 2) : 1.f; o.out_scale = f8 ? act_scale(l, 3) : 1.f; o.amax = am(l, 3);
          RUN(gemm(ly.ff1, h_in, C, ao_dt, f8 ? (void*)ws.f8 : (void*)ws.f, F, ao_dt, M, o, st)); }
        { GOpt o; o.act = ACT_GELU; o.res = ws.h; o.ldr = C; o.res_dt = xdt; o.a_scale = f8 ? act_scale(l, 3) : 1.f;
          RUN(gemm(ly.ff2, f8 ? (const void*)ws.f8 : (const void*)ws.f, F, ao_dt, ws.t, C, xdt, M, o, st)); }
      } else {
        { GOpt o; o.act = ACT_MISH; o.a_scale = f8 ? act_scale(l, 2) : 1.f; o.out_scale = f8 ? act_scale(l, 3) : 1.f; o.amax = am(l, 3);
          RUN(gemm(ly.ff1, h_in, C, ao_dt, f8 ? (void*)ws.f8 : (void*)ws.f, F, ao_dt, M, o, st)); }
        { GOpt o; o.res = ws.h; o.ldr = C; o.res_dt = xdt; o.alpha = alpha; o.a_scale = f8 ? act_scale(l, 3) : 1.f;
          if (fold) { o.res = ws.t; o.res_stats = ws.st1; o.res_g = ly.ln1_g; o.res_b = ly.ln1_b; }
          RUN(gemm(ly.ff2, f8 ? (const void*)ws.f8 : (const void*)ws.f, F, ao_dt, ws.t, C, xdt, M, o, st)); }
      }
      // x = LN2(t); the last layer's output feeds only the heads (as an e4m3 copy alone when they run in e4m3).
      const bool x8_out = f8 && (!last || f8h);
      RUN(lnorm(ws.t, C, xdt, ly.ln2_g, ly.ln2_b, ((fold && !last) || (last && f8h)) ? nullptr : ws.x, last ? hd : xdt, x8_out ? ws.x8 : nullptr,
                x8_out ? act_scale(l + 1, 0) : 1.f, C, M, C, (last && !cal_heads) ? nullptr : am(l + 1, 0), st, (fold && !last) ? ws.st2 : nullptr,
                (sf32p && !f8 && !last) ? ws.x16 : nullptr, ad));
    }
  }

  if (win) {
    HIPCHK(launch_widen(ws.x, gpt ? xdt : hd, win->x_out, (long)M * C, st));
    return CRL_OK;
  }

  // ---- heads
  if (gpt) {
    // lm_head takes e4m3 operands too in the fp8 model (model_fp8.py:140); its input scale is the first entry of the
    // amax table's last row.
    // An uncalibrated head row (a legacy n_layer*5 table was loaded) keeps lm_head on its 16-bit copy.
    const bool f8h = f8 && lm_head.w8 != nullptr && amax_host[(size_t)L * AMAX_SLOTS] > 0.f;
    const float hsc = f8h ? act_scale(L, 0) : 1.f;
    // Calibration takes the head's input amax over EVERY token of ln_f: forward_tokens(all_logits) quantises all of them
    // with this one scale (model_bis.py:189-192), not just the last token that the policy-only forward reads.
    const bool cal_all = calibrate && !all_logits;
    if (cal_all) RUN(lnorm(ws.x, C, xdt, lnf_g, lnf_b, ws.h, hd, nullptr, 1.f, C, M, C, am(L, 0), st));
    if (all_logits) {
      // ln_f and lm_head on every token (model_bis.py:189-192, compute_loss=True).
      RUN(lnorm(ws.x, C, xdt, lnf_g, lnf_b, f8h ? nullptr : ws.h, hd, f8h ? ws.h8 : nullptr, hsc, C, M, C, am(L, 0), st));
      GOpt o; o.a_scale = hsc;
      RUN(gemm(lm_head, f8h ? (const void*)ws.h8 : (const void*)ws.h, C, f8h ? DT_FP8 : hd, all_logits, VOCAB_RL, DT_F32, M, o, st));
    }
    if (policy) {
      // ln_f and lm_head on the last token only (model_bis.py:195-196, 369-370).
      const char* last_tok = reinterpret_cast<const char*>(ws.x) + (size_t)(T - 1) * C * dtype_size(xdt);
      RUN(lnorm(last_tok, (long)T * C, xdt, lnf_g, lnf_b, f8h ? nullptr : ws.hl, hd, f8h ? ws.hl8 : nullptr, hsc, C, mb, C, nullptr, st));
      GOpt o; o.a_scale = hsc;
      RUN(gemm(lm_head, f8h ? (const void*)ws.hl8 : (const void*)ws.hl, C, f8h ? DT_FP8 : hd, policy, VOCAB_RL, DT_F32, mb, o, st));
    }
    return CRL_OK;
  }
  const int hact = cfg.arch == CRL_ARCH_BT4 ? ACT_GELU : ACT_MISH;
  const void* x_head = f8h ? (const void*)ws.x8 : (const void*)ws.x;
  const int xh_dt = f8h ? DT_FP8 : hd;
  const float xh_sc = f8h ? act_scale(L, 0) : 1.f;
  if (wdl) {
    { GOpt o; o.act = hact; o.a_scale = xh_sc; RUN(gemm(val1, x_head, C, xh_dt, ws.v1, 128, hd, M, o, st)); }
    { GOpt o; o.act = hact; RUN(gemm(val2, ws.v1, 8192, hd, ws.v2, 128, hd, mb, o, st)); }
    { GOpt o; RUN(gemm(val3, ws.v2, 128, hd, wdl, 3, DT_F32, mb, o, st)); }
  }
  {
    GOpt o; o.act = hact;
    if (cfg.arch == CRL_ARCH_BT4) { o.res = pe_head; o.ldr = C; o.res_dt = hd; o.res_rows = 64; }
    o.a_scale = xh_sc;
    if (f8h) o.out_scale = act_scale(L, 1);
    if (cal_heads) o.amax = am(L, 1);
    // (the e4m3 policy tokens take the place of h8, which nothing reads after the trunk)
    RUN(gemm(pol_tok, x_head, C, xh_dt, f8h ? (void*)ws.h8 : ws.tok, C, f8h ? DT_FP8 : hd, M, o, st));
  }
  { GOpt o; o.a_scale = f8h ? act_scale(L, 1) : 1.f;
    RUN(gemm(pol_qk, f8h ? (const void*)ws.h8 : (const void*)ws.tok, C, xh_dt, ws.pqk, 2 * C, hd, M, o, st)); }
  {
    PolicyQKArgs p;
    std::memset(&p, 0, sizeof(p));
    const uint16_t* base = reinterpret_cast<const uint16_t*>(ws.pqk);
    p.q = base; p.k = base + C; p.ldq = p.ldk = 2 * C; p.in_dtype = hd; p.B = mb; p.C = C;
    p.scale = 1.0f / std::sqrt((float)C);
    if (cfg.arch == CRL_ARCH_BT4) { p.dense = ws.dense; p.dense_dtype = hd; p.ldd = 4096; }
    else { p.logits = policy; p.ldl = VOCAB_LEELA; p.gidx = gidx; p.gpromo = gpromo; p.wpromo = promo_w; p.white_to_move = ws.stm; p.nmoves = VOCAB_LEELA; }
    prof_begin(4, st);
    hipError_t he = launch_policy_qk(p, st);
    prof_end(st);
    HIPCHK(he);
  }
  if (cfg.arch == CRL_ARCH_BT4) { GOpt o; RUN(gemm(pol_head, ws.dense, 4096, hd, policy, VOCAB_RL, DT_F32, mb, o, st)); }
#undef RUN
  return CRL_OK;
}

int Model::run_layers(const float* x_in, int B, int first, int last, float* x_out, hipStream_t st) {
  if (!finalized) { set_error("run_layers: call crl_model_finalize first"); return CRL_ERR_STATE; }
  if (cfg.arch != CRL_ARCH_BT4CLASS) { set_error("run_layers: only CRL_ARCH_BT4CLASS has a layer-window entry"); return CRL_ERR_ARG; }
  if (!x_in || !x_out || B <= 0 || first < 0 || last > cfg.n_layer || first >= last) { set_error("run_layers: bad arguments (0 <= first < last <= n_layer)"); return CRL_ERR_ARG; }
  if (B > cfg.micro_batch) { set_error("run_layers: at most one micro-batch of positions"); return CRL_ERR_ARG; }
  int rc = ensure_ws(B);
  if (rc) return rc;
  LayerWindow w{first, last, x_in, x_out};
  float dummy_policy;   // never written: the window returns before the heads
  return forward_chunk(nullptr, nullptr, nullptr, nullptr, 0, B, &dummy_policy, nullptr, nullptr, false, st, &w);
}

int Model::debug_read(const char* name, void* out, long bytes, hipStream_t st) {
  if (!name || !out || bytes < 0 || ws_mb == 0) { set_error("debug_read: bad arguments, or no forward has run yet"); return CRL_ERR_ARG; }
  const size_t M = (size_t)ws_mb * 64, C = cfg.d_model, F = cfg.d_ff;
  const std::string n = name;
  const void* src = nullptr;
  size_t cap = 0;
  if (n == "x8") { src = ws.x8; cap = M * C; }
  else if (n == "h8") { src = ws.h8; cap = M * C; }
  else if (n == "ao8") { src = ws.ao8; cap = M * C; }
  else if (n == "f8") { src = ws.f8; cap = M * F; }
  else if (n == "t") { src = ws.t; cap = M * C * ((cfg.arch != CRL_ARCH_GPT64 && cfg.stream_f32 > 0) ? 4 : 2); }
  else { set_error("debug_read: unknown tensor " + n); return CRL_ERR_ARG; }
  if ((size_t)bytes > cap) { set_error("debug_read: " + n + " holds " + std::to_string(cap) + " bytes"); return CRL_ERR_ARG; }
  HIPCHK(hipMemcpyAsync(out, src, (size_t)bytes, hipMemcpyDeviceToDevice, st));
  return CRL_OK;
}

int Model::calibrate(const float* planes, int B, hipStream_t st) {
  if (!finalized) { set_error("calibrate: call crl_model_finalize first"); return CRL_ERR_STATE; }
  HIPCHK(launch_fill_f32(amax_dev, 0.f, (long)amax_host.size(), st));
  float* pol = nullptr;
  HIPCHK(hipMalloc((void**)&pol, (size_t)B * vocab * sizeof(float)));
  int rc = forward(planes, nullptr, nullptr, B, pol, nullptr, true, st);
  hipError_t e = hipStreamSynchronize(st);
  if (rc == CRL_OK && e == hipSuccess) e = hipMemcpy(amax_host.data(), amax_dev, sizeof(float) * amax_host.size(), hipMemcpyDeviceToHost);
  (void)hipFree(pol);
  if (rc) return rc;
  HIPCHK(e);
  return CRL_OK;
}

int Model::generate(const float* planes, int B, int steps, float temperature, uint64_t seed, int rules, int64_t* seq, float* step_out,
                    int out_logits, hipStream_t st) {
  if (!finalized) { set_error("generate: call crl_model_finalize first"); return CRL_ERR_STATE; }
  if (cfg.arch != CRL_ARCH_GPT64) { set_error("generate: only CRL_ARCH_GPT64 generates sequences"); return CRL_ERR_ARG; }
  if (!planes || !seq || B <= 0 || steps < 1 || temperature < 0.f) { set_error("generate: bad arguments"); return CRL_ERR_ARG; }
  const int C = cfg.d_model, F = cfg.d_ff, H = cfg.n_head, L = cfg.n_layer, hs = C / H;
  const int Tmax = 64 + steps;   // the last sampled token is never fed back
  if (Tmax > pe_rows || Tmax > 1024) { set_error("generate: 64 + steps exceeds the positional table or 1024 tokens"); return CRL_ERR_ARG; }
  if ((long)B * 65 > (long)cfg.micro_batch * 64) { set_error("generate: batch too large for one micro-batch"); return CRL_ERR_ARG; }
  int rc = ensure_ws((int)(((long)B * 65 + 63) / 64));
  if (rc) return rc;
  if (B > kv_B || Tmax > kv_Tmax || (int)kv_layers.size() != L) {
    for (void* p : gen_allocs) (void)hipFree(p);
    gen_allocs.clear();
    kv_layers.assign(L, nullptr);
    kv_B = kv_Tmax = 0;
    auto galloc = [&](void** p, size_t bytes) -> int {
      hipError_t e = hipMalloc(p, bytes ? bytes : 16);
      if (e != hipSuccess) { set_error(std::string("generate: ") + hipGetErrorString(e)); return CRL_ERR_HIP; }
      gen_allocs.push_back(*p);
      return CRL_OK;
    };
    for (int l = 0; l < L; ++l) { rc = galloc(&kv_layers[l], (size_t)B * Tmax * 2 * C * 2); if (rc) return rc; }
    rc = galloc((void**)&gen_tok, sizeof(int64_t) * B); if (rc) return rc;
    rc = galloc((void**)&gen_zeros, sizeof(int32_t) * B); if (rc) return rc;
    rc = galloc((void**)&gen_logits, sizeof(float) * (size_t)B * VOCAB_RL); if (rc) return rc;
    rc = galloc((void**)&gen_kv_stage, (size_t)B * 2 * C * 2); if (rc) return rc;
    rc = galloc((void**)&gen_k, 256); if (rc) return rc;
    kv_B = B; kv_Tmax = Tmax;
  }
  const int hd = cfg.head_dtype, ad = cfg.act_dtype;
  const int xdt = cfg.stream_f32 > 0 ? DT_F32 : ad;
  const long START_THINK = 1924, END_THINK = 1925, END_VARIATION = 1926, END = 1927;
  // <thinking> opens every sequence (model_bis.py:221-224); gen_zeros doubles as the fill source via a tiny host copy.
  {
    std::vector<int64_t> first(B, START_THINK);
    std::vector<int32_t> zeros(B, 0);
    const int first_replayed = 2;
    HIPCHK(hipMemcpyAsync(gen_k, &first_replayed, sizeof(int), hipMemcpyHostToDevice, st));
    HIPCHK(hipMemcpyAsync(gen_tok, first.data(), sizeof(int64_t) * B, hipMemcpyHostToDevice, st));
    HIPCHK(hipMemcpyAsync(gen_zeros, zeros.data(), sizeof(int32_t) * B, hipMemcpyHostToDevice, st));
    HIPCHK(hipMemcpy2DAsync(seq, sizeof(int64_t) * (steps + 1), gen_tok, sizeof(int64_t), sizeof(int64_t), B, hipMemcpyDeviceToDevice, st));
    HIPCHK(hipStreamSynchronize(st));   // the host vectors go out of scope
  }
#define RUN(call) do { rc = (call); if (rc) { kv_capture = false; force_16bit = false; return rc; } } while (0)
  // Prefix of 65 tokens: fills the cache and gives the logits of the first sampled token.
  kv_capture = true; force_16bit = true;
  RUN(forward_chunk(planes, nullptr, nullptr, gen_tok, 1, B, gen_logits, nullptr, nullptr, false, st));
  kv_capture = false;
  const float attn_scale = 1.0f / std::sqrt((float)hs);
  // One token step: sample token k from gen_logits, then (unless it is the last) run it through the trunk at position
  // 64 + k against the cache and leave the next logits in gen_logits. With `dyn` the kernels read k from device memory
  // and the step ends by advancing it, so the same launches serve every k (the body of the replayed graph).
  auto token_step = [&](int k, const int* dyn, bool sample_only, hipStream_t s) -> int {
    int rc = CRL_OK;
#define STEP_HIP(expr) do { hipError_t he_ = (expr); if (he_ != hipSuccess) { set_error(std::string("generate: ") + hipGetErrorString(he_)); return CRL_ERR_HIP; } } while (0)
#define STEP_RUN(call) do { rc = (call); if (rc) return rc; } while (0)
    SampleArgs sa;
    std::memset(&sa, 0, sizeof(sa));
    sa.logits = gen_logits; sa.ldl = VOCAB_RL; sa.seq = seq; sa.ld_seq = steps + 1; sa.tok_out = gen_tok; sa.num_zeros = gen_zeros;
    sa.step_out = !step_out ? nullptr : dyn ? step_out : step_out + (size_t)(k - 1) * VOCAB_RL;
    sa.ld_out = (long)steps * VOCAB_RL;
    sa.B = B; sa.V = VOCAB_RL; sa.k = k; sa.step = k; sa.rules = rules; sa.out_logits = out_logits; sa.dyn_k = dyn;
    sa.end_think = END_THINK; sa.end_tok = END; sa.end_variation = END_VARIATION; sa.temperature = temperature; sa.seed = seed;
    STEP_HIP(launch_sample(sa, s));
    if (sample_only) return CRL_OK;
    const int pos = 64 + k;    // sequence position of token k
    STEP_HIP(launch_decode_embed(gen_tok, wte_f32, pe_f32, pos, dyn, ws.x, B, C, VOCAB_RL, xdt, s));
    bool normed = false;   // ws.h (or, after the last layer, ws.hl) already holds the next LayerNorm's output
    for (int l = 0; l < L; ++l) {
      const Layer& ly = layers[l];
      if (!normed) STEP_RUN(lnorm(ws.x, C, xdt, ly.ln1_g, ly.ln1_b, ws.h, ad, nullptr, 1.f, C, B, C, nullptr, s));
      if (dyn) {
        // q -> ws.qkv [B,C]; k|v -> staging, then to the row the counter names
        GOpt o; o.k_parallel = true; o.C2 = gen_kv_stage; o.ldc2 = 2 * C; o.nsplit = C;
        STEP_RUN(gemm(ly.qkv, ws.h, C, ad, ws.qkv, C, ad, B, o, s));
        STEP_HIP(launch_kv_append(gen_kv_stage, kv_layers[l], B, kv_Tmax, C, 0, dyn, s));
      } else {
        // q -> ws.qkv [B,C]; k|v -> row `pos` of every sequence's cache
        GOpt o; o.k_parallel = true; o.C2 = reinterpret_cast<uint16_t*>(kv_layers[l]) + (size_t)pos * 2 * C; o.ldc2 = (long)kv_Tmax * 2 * C; o.nsplit = C;
        STEP_RUN(gemm(ly.qkv, ws.h, C, ad, ws.qkv, C, ad, B, o, s));
      }
      STEP_HIP(launch_decode_attention(ws.qkv, C, kv_layers[l], kv_Tmax, C, pos + 1, dyn, ws.ao, C, B, H, hs, ad, attn_scale, s));
      bool normed2 = false;
      { GOpt o; o.k_parallel = true; o.res = ws.x; o.ldr = C; o.res_dt = xdt;
        o.ln_g = ly.ln2_g; o.ln_b = ly.ln2_b; o.ln_out = ws.h; o.ln_dt = ad; o.ln_folded = &normed2;
        STEP_RUN(gemm(ly.proj, ws.ao, C, ad, ws.x, C, xdt, B, o, s)); }
      if (!normed2) STEP_RUN(lnorm(ws.x, C, xdt, ly.ln2_g, ly.ln2_b, ws.h, ad, nullptr, 1.f, C, B, C, nullptr, s));
      { GOpt o; o.k_parallel = true; o.act = ACT_GELU; STEP_RUN(gemm(ly.ff1, ws.h, C, ad, ws.f, F, ad, B, o, s)); }
      { // the norm that reads this GEMM's result (the next layer's ln_1, or ln_f) rides on its second pass where it is K-sliced
        GOpt o; o.k_parallel = true; o.res = ws.x; o.ldr = C; o.res_dt = xdt; o.ln_folded = &normed;
        if (l + 1 < L) { o.ln_g = layers[l + 1].ln1_g; o.ln_b = layers[l + 1].ln1_b; o.ln_out = ws.h; o.ln_dt = ad; }
        else { o.ln_g = lnf_g; o.ln_b = lnf_b; o.ln_out = ws.hl; o.ln_dt = hd; }
        STEP_RUN(gemm(ly.ff2, ws.f, F, ad, ws.x, C, xdt, B, o, s)); }
    }
    if (!normed) STEP_RUN(lnorm(ws.x, C, xdt, lnf_g, lnf_b, ws.hl, hd, nullptr, 1.f, C, B, C, nullptr, s));
    { GOpt o; o.k_parallel = true; STEP_RUN(gemm(lm_head, ws.hl, C, hd, gen_logits, VOCAB_RL, DT_F32, B, o, s)); }
    if (dyn) STEP_HIP(launch_add_int(gen_k, 1, s));
    return CRL_OK;
#undef STEP_HIP
#undef STEP_RUN
  };
  // Steps 2 .. steps-1 are identical launches apart from k: they are recorded once and replayed, which takes the host's
  // launch cost (some 8 launches per layer) off the critical path. Step 1 runs eagerly first so that every kernel's
  // one-time set-up has happened before the recording; the timers of the profiling mode cannot be recorded, so that
  // mode stays on plain launches.
  const bool graphed = decode_graph && !profiling && steps >= 4;
  int k = 1;
  if (graphed) {
    RUN(token_step(1, nullptr, false, st));
    if (!cap_stream) HIPCHK(hipStreamCreateWithFlags(&cap_stream, hipStreamNonBlocking));
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipError_t he = hipStreamBeginCapture(cap_stream, hipStreamCaptureModeRelaxed);
    if (he != hipSuccess) { force_16bit = false; HIPCHK(he); }
    rc = token_step(2, gen_k, false, cap_stream);
    he = hipStreamEndCapture(cap_stream, &graph);   // always ends the recording, also after a failed launch
    if (rc == CRL_OK && he == hipSuccess) he = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    for (k = 2; rc == CRL_OK && he == hipSuccess && k < steps; ++k) he = hipGraphLaunch(exec, st);
    if (rc == CRL_OK && he == hipSuccess) he = hipStreamSynchronize(st);   // the graph is destroyed below
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (rc) { force_16bit = false; return rc; }
    if (he != hipSuccess) { force_16bit = false; HIPCHK(he); }
    k = steps;
  }
  for (; k <= steps; ++k) RUN(token_step(k, nullptr, k == steps, st));
#undef RUN
  force_16bit = false;
  prof_collect(st);
  return CRL_OK;
}

double Model::flops_per_position() const {
  const double T = 64, C = cfg.d_model, F = cfg.d_ff, L = cfg.n_layer, H = cfg.n_head;
  if (cfg.arch == CRL_ARCH_GPT64)
    return L * (8 * T * C * C + 4 * T * C * F + 2 * T * (T + 1) * C) + 2 * T * 19 * C + 2 * C * VOCAB_RL;
  const double heads_common = 2 * T * C * 128 + 2 * 8192.0 * 128 + 2 * 128 * 3 + 2 * T * 19 * C;
  if (cfg.arch == CRL_ARCH_BT4)
    return L * (8 * T * C * C + 6 * T * T * C + 4 * T * C * F) + 6 * T * C * C + 2 * T * T * C + 2 * 4096.0 * VOCAB_RL + heads_common;
  const double sc = cfg.smolgen_compress, sh = cfg.smolgen_hidden, sg = cfg.smolgen_gen;
  const double smol = 2 * T * C * sc + 2 * 64 * sc * sh + 2 * sh * H * sg + 2 * H * sg * 4096;
  return L * (8 * T * C * C + 4 * T * T * C + 4 * T * C * F + smol) + 6 * T * C * C + 2 * T * T * C + 2 * 8 * 4 * C + heads_common;
}

}  // namespace crl
