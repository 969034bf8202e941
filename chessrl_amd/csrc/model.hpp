// Host-side model runner (see model.hip).
#pragma once
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "../../include/chessrl_amd.h"
#include "host/chess.hpp"
#include "kernels/common.hpp"

namespace crl {

void set_error(const std::string& s);
const char* get_error();

// One linear layer on the device: a 16-bit copy, an optional e4m3 copy (value*wscale)
// and an fp32 bias.
struct Lin {
  void* w = nullptr;
  void* w8 = nullptr;
  float* b = nullptr;
  int N = 0, K = 0, dt = DT_BF16;
  float wscale = 1.f;
};

struct Layer {
  Lin qkv, proj, ff1, ff2, sm_hidden, sm_gen;
  float *ln1_g = nullptr, *ln1_b = nullptr, *ln2_g = nullptr, *ln2_b = nullptr;
  float *sm_ln1_g = nullptr, *sm_ln1_b = nullptr, *sm_ln2_g = nullptr, *sm_ln2_b = nullptr;
  void* pos = nullptr;
  float *u_bias = nullptr, *v_bias = nullptr;
};

struct Workspace {
  void *x = nullptr, *t = nullptr, *h = nullptr, *qkv = nullptr, *ao = nullptr, *f = nullptr;
  void *x16 = nullptr, *h16 = nullptr;   // 16-bit operand copies of x and h beside an fp32 residual stream (BT4, BT4-class)
  uint8_t* hl8 = nullptr;                // e4m3 input of lm_head
  uint8_t *x8 = nullptr, *h8 = nullptr, *ao8 = nullptr, *f8 = nullptr, *stm = nullptr;
  float *st1 = nullptr, *st2 = nullptr;   // row statistics (mean, 1/std) of a layer's two LayerNorms
  void *comp = nullptr, *sh1 = nullptr, *sh2 = nullptr, *sg1 = nullptr, *sg2 = nullptr, *bias = nullptr;
  uint8_t* sg2_8 = nullptr;
  void *hl = nullptr, *tok = nullptr, *pqk = nullptr, *v1 = nullptr, *v2 = nullptr, *dense = nullptr;
  float* splitk = nullptr;    // partial tiles of the K-sliced GEMMs (SPLITK_BYTES)
  static constexpr long SPLITK_BYTES = 64L << 20;
};

struct GOpt;

// A run of consecutive encoder layers on a caller-supplied input (Model::run_layers).
struct LayerWindow {
  int first, last;
  const float* x_in;   // device f32 [positions*64, d_model]: input of layer `first`
  float* x_out;        // device f32, same shape: output of layer `last - 1`
};

struct Model {
  // q and k columns of the concatenated q|k|v weight paired head by head (BT4-class with 64-byte head rows)
  bool qk_paired() const { return cfg.arch == CRL_ARCH_BT4CLASS && cfg.d_model / cfg.n_head == 32; }
  crl_model_config cfg;
  int vocab = 0;
  bool finalized = false;
  std::vector<std::pair<std::string, long>> expected;
  std::map<std::string, std::vector<float>> host;

  std::vector<void*> allocs, ws_allocs;
  std::vector<Layer> layers;
  float *emb_w1t = nullptr, *emb_b1 = nullptr, *emb_g = nullptr, *emb_b = nullptr, *gate_a_exp = nullptr, *gate_b = nullptr;
  float *pe_f32 = nullptr, *wte_f32 = nullptr, *lnf_g = nullptr, *lnf_b = nullptr, *promo_w = nullptr;
  int pe_rows = 0;
  void* pe_head = nullptr;
  Lin lm_head, pol_tok, pol_qk, pol_head, val1, val2, val3, sm_weight_gen;
  int16_t* gidx = nullptr;
  int8_t* gpromo = nullptr;
  // Activation amax table [n_layer + 1][AMAX_SLOTS]: input of q|k|v, attention output, input of FFN-1, input of FFN-2,
  // input of the shared bias generator (BT4-class only); the first entry of the last row is the input of lm_head (GPT64).
  static constexpr int AMAX_SLOTS = 5;
  float* amax_dev = nullptr;
  std::vector<float> amax_host;
  Workspace ws;
  int ws_mb = 0;
  // generation state, grown on demand: per layer [B, Tmax, 2C] 16-bit keys|values, newest tokens, counters, logits
  std::vector<void*> kv_layers;
  std::vector<void*> gen_allocs;
  int kv_B = 0, kv_Tmax = 0;
  int64_t* gen_tok = nullptr;
  int32_t* gen_zeros = nullptr;
  float* gen_logits = nullptr;
  void* gen_kv_stage = nullptr;     // [B, 2C] k|v of the newest token inside a replayed step
  int* gen_k = nullptr;             // device counter: index of the token a replayed step samples
  hipStream_t cap_stream = nullptr; // records the step graph (nothing executes on it)
  bool decode_graph = false;
  bool kv_capture = false;     // forward_chunk copies every layer's keys|values into the cache
  bool force_16bit = false;    // forward_chunk ignores cfg.fp8

  struct ProfEvent { hipEvent_t a, b; int fam; };
  bool profiling = false;
  std::vector<ProfEvent> prof_events;
  size_t prof_used = 0;
  double prof_ms[6] = {0, 0, 0, 0, 0, 0};
  double prof_flops[6] = {0, 0, 0, 0, 0, 0};
  long prof_n[6] = {0, 0, 0, 0, 0, 0};

  explicit Model(const crl_model_config& c);
  ~Model();
  int set_weight(const char* key, const float* data, long numel);
  int finalize();
  int forward(const float* planes, const uint8_t* ids, const uint8_t* flags, int B, float* policy, float* wdl, bool calibrate, hipStream_t st);
  // CRL_ARCH_GPT64 with t move tokens after the 64 board tokens; policy = logits of the last token [B,V],
  // all_logits = logits of every token [B, 64+t, V]; either may be null.
  int forward_tokens(const float* planes, const uint8_t* ids, const uint8_t* flags, const int64_t* idx, int t, int B, float* policy,
                     float* all_logits, float* wdl, bool calibrate, hipStream_t st);
  int calibrate(const float* planes, int B, hipStream_t st);
  // Layers [first, last) on x_in (device f32 [B*64, d_model]); x_out receives the output of layer last-1 widened to f32.
  // The window's first layer takes x_in as its residual as layer 0 takes the embedding, its last layer writes its
  // normalised output in the 16-bit type as the trunk's last layer does; everything between runs as in forward().
  int run_layers(const float* x_in, int B, int first, int last, float* x_out, hipStream_t st);
  // Copies a workspace tensor as the last call left it ("x8", "h8", "ao8", "f8": the e4m3 operand copies; "t") to `out`.
  int debug_read(const char* name, void* out, long bytes, hipStream_t st);
  // Sequence generation with cached keys/values (model_bis.py:213-263 with rules, 266-311 without): seq [B, steps+1]
  // receives <thinking> and then `steps` sampled tokens; step_out [B, steps, V] (optional) the probabilities of
  // every step, or its logits when out_logits. Runs in the 16-bit element type whatever cfg.fp8 says.
  int generate(const float* planes, int B, int steps, float temperature, uint64_t seed, int rules, int64_t* seq, float* step_out,
               int out_logits, hipStream_t st);
  double flops_per_position() const;

 private:
  const std::vector<float>& w(const std::string& k);
  int dev_alloc(void** p, size_t bytes, bool ws);
  int upload(const std::vector<float>& v, int dt, float scale, void** out);
  int make_lin(Lin& L, const std::vector<float>& W, const std::vector<float>* bias, int N, int K, int dt16, bool fp8, float amax_all = -1.f);
  int ensure_ws(int mb);
  int forward_chunk(const float* planes, const uint8_t* ids, const uint8_t* flags, const int64_t* idx, int t, int mb, float* policy,
                    float* all_logits, float* wdl, bool calibrate, hipStream_t st, const LayerWindow* win = nullptr);
  int gemm(const Lin& L, const void* A, long lda, int in_dt, void* C, long ldc, int out_dt, int M, const GOpt& o, hipStream_t st);
  int lnorm(const void* x, long ldx, int in_dt, const float* g, const float* b, void* out, int out_dt, uint8_t* out8, float scale8,
            long ldo, int rows, int C, float* amax, hipStream_t st, float* stats = nullptr, void* out_b = nullptr, int out_b_dt = DT_BF16,
            bool trunk = true);
  float act_scale(int layer, int slot) const;
  void prof_begin(int fam, hipStream_t st);
  void prof_end(hipStream_t st);
  void prof_collect(hipStream_t st);
};

}  // namespace crl
