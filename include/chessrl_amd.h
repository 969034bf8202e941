/* chessrl_amd — C ABI of the MI355X (gfx950) policy/value forward path.
 *
 * The reference (maxlegrec1/ChessRL) has no FFI layer: its boundary for this path is
 * the Python nn.Module surface plus the state-dict. Every entry point below therefore
 * cites the reference Python interface it stands in for; chessrl_amd/models.py is the
 * ctypes binding that rebuilds that surface on top of this header.
 *
 * Conventions: every function returns 0 on success and a negative code on failure
 * (crl_last_error() gives the message for the calling thread). No exception crosses
 * the boundary. "device" pointers are HIP device pointers owned by the caller (for
 * example torch tensors' data_ptr()); "stream" is a hipStream_t passed as void*
 * (NULL = the default stream). The library never synchronises the stream unless the
 * function says so. Host-only functions touch no GPU state and work without a GPU.
 */
#ifndef CHESSRL_AMD_H
#define CHESSRL_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CRL_OK 0
#define CRL_ERR_ARG (-1)      /* bad argument / shape / alignment */
#define CRL_ERR_HIP (-2)      /* a HIP call failed */
#define CRL_ERR_STATE (-3)    /* call order (e.g. forward before finalize, missing weight) */
#define CRL_ERR_FEN (-4)      /* malformed FEN */

#define CRL_VOCAB_RL 1929     /* utils/vocab.py:9-227   policy_index */
#define CRL_VOCAB_LEELA 1858  /* utils/vocab.py:229-438 policy_leela */
#define CRL_NUM_PLANES 19     /* utils/fen_encoder.py:7 */

/* element types */
#define CRL_F32 0
#define CRL_BF16 1
#define CRL_F16 2
#define CRL_FP8 3             /* OCP e4m3fn */
/* activations */
#define CRL_ACT_NONE 0
#define CRL_ACT_GELU 1        /* erf form, nn.GELU() */
#define CRL_ACT_MISH 2
#define CRL_ACT_SWISH 3
/* attention modes */
#define CRL_ATTN_PLAIN 0
#define CRL_ATTN_CAUSAL 1     /* model_bis.py:71 */
#define CRL_ATTN_BIAS 2       /* generated per-head 64x64 bias (BT4-class) */
#define CRL_ATTN_RELSHIFT 3   /* new_paradigm/attn.py:507-533 */
/* model architectures */
#define CRL_ARCH_GPT64 0      /* model_bis.GPT, 64-token forward (model_bis.py:358-370) */
#define CRL_ARCH_BT4 1        /* new_paradigm/value.py BT4 */
#define CRL_ARCH_BT4CLASS 2   /* BT4-class encoder of the benchmark configuration */

const char* crl_last_error(void);
const char* crl_version(void);
/* Frees the device memory the library keeps outside any model handle: the 64 MB K-slice workspaces crl_gemm allocates per
 * stream, a 256-byte block of zeros per device and the move maps of crl_leela_to_rl. Call it with no library work in
 * flight; later calls allocate again on demand. Models are freed by crl_model_destroy. A HIP graph captured from
 * library calls has those device addresses baked in: destroy or re-capture such graphs after crl_shutdown. */
void crl_shutdown(void);

/* ------------------------------------------------------------------ host: vocabulary */
/* utils/vocab.py:9-227 / :229-438 — i-th move string (static storage), NULL if out of range. */
const char* crl_policy_index(int i);
const char* crl_policy_leela(int i);
/* policy_index.index(uci) with the reference's trailing-'n' strip (model_bis.py:376-380); -1 if absent. */
int crl_move_to_index(const char* uci);
/* Leela/compare_policy.py:470-491 — mapping_white / mapping_black, int32[1858] each. */
int crl_leela_to_rl_maps(int32_t* white_out, int32_t* black_out);

/* ------------------------------------------------------------------ host: boards */
/* utils/fen_encoder.py:5-38 fen_to_tensor: float32[64*19] in token order t=(7-rank)*8+file. */
int crl_fen_to_planes(const char* fen, float* out_planes);
/* utils/parse.py:71-75 encode_fens: n FENs -> float32[n,64,19]; threads<=0 picks a default. */
int crl_encode_fens(const char* const* fens, int n, float* out_planes, int threads);
/* Compact form of the same information: uint8[n,64] piece codes (0 empty, 1..6 PNBRQK,
 * 7..12 pnbrqk) and uint8[n,4] {white_to_move, castling bits WK|WQ<<1|BK<<2|BQ<<3,
 * en-passant token or 255, min(halfmove,100)}. */
int crl_encode_fens_compact(const char* const* fens, int n, uint8_t* out_ids, uint8_t* out_flags, int threads);
/* model_bis.py:373-380 (same code grpo_refactored.py:374-384, new_paradigm/value.py:222-231):
 * uint8[n,1929] legal-move masks; out_counts (optional) gets len(list(board.legal_moves)). */
int crl_legal_masks(const char* const* fens, int n, uint8_t* out_masks, int32_t* out_counts, int threads);
/* Same for the 1858-entry side-to-move frame (black rows rank-mirrored, Leela/compare_policy.py:437-463). */
int crl_legal_masks_leela(const char* const* fens, int n, uint8_t* out_masks, int32_t* out_counts, int threads);
/* Legal moves of one position as UCI strings, 6 bytes each (NUL padded), in generation
 * order; returns the count (<= max_moves) or a negative code. new_paradigm/value.py:331. */
int crl_legal_moves(const char* fen, char* out_uci6, int max_moves);
/* board.push(move); board.fen() for every legal move (new_paradigm/value.py:336-340):
 * writes child FENs (96 bytes each, NUL terminated) and the moves (6 bytes each). */
int crl_child_fens(const char* fen, char* out_fens96, char* out_uci6, int max_moves);
uint64_t crl_perft(const char* fen, int depth);
/* Seeded uniform-random legal playouts from the start position (splitmix64): position k
 * gets U{0..max_plies} plies; when late_fraction>0 that share of positions is instead
 * played on until at most late_max_pieces pieces remain. Outputs (each optional):
 * float32[n,64,19] planes, uint8[n,1929] masks, uint8[n,1858] masks, FENs (96 bytes each). */
int crl_random_positions(uint64_t seed, int n, int max_plies, double late_fraction, int late_max_pieces,
                         float* out_planes, uint8_t* out_masks_rl, uint8_t* out_masks_leela, char* out_fens96);

/* ------------------------------------------------------------------ device: operators */
/* nn.Linear / te.Linear (model_bis.py:42-44,89-91,139; model_fp8.py:43-45,90-92,140;
 * new_paradigm/value.py:39-40,129-152): C = res + alpha*act(descale*(A·W^T) + bias).
 * A [M,K] (lda), W [N,K] (ldw) of in_dtype (bf16/f16/fp8); C [M,N] (ldc) of out_dtype;
 * bias fp32[N] or NULL; res [M,N] of res_dtype (f32/bf16) or NULL; for an fp8 output the
 * value is multiplied by out_scale before conversion; amax (device float, optional)
 * accumulates max|value|. tile: 0 = automatic among 1-3 = the 64x64 / 128x128 / 256x256 workgroup tile; these add up
 * K in one order, so a row's result does not depend on the other rows of the call. For few rows (the token steps of
 * crl_model_generate use them): 4 = 64x64 tiles with K cut into slices, one workgroup per (tile, slice) leaving raw
 * fp32 sums in a workspace of 64 MB that the library keeps per stream, and a second kernel that adds them in slice
 * order and applies the epilogue; 5 = 64x64 tiles whose K slabs four groups of four waves take in turn and add up in
 * LDS. Both are deterministic from launch to launch but differ from 1-3 in summation order. With tile 0, outputs of at
 * most 256 columns whose K is 8 KB or more per row are always K-sliced the same way (a function of N and K alone), so
 * the row-count independence holds for them too. The first K-sliced launch on a stream allocates that stream's
 * workspace: issue it once outside any graph capture. 7, 9 and 10 name the 256x256 kernels explicitly: 7 = eight waves in
 * step (any K, any operand type), 10 = the same with its address arithmetic kept out of the main loop (K in whole
 * 128-byte slabs; 3 runs this one where it applies), both with the sums and result bits of 1-3; 9 = four
 * software-pipelined waves with 16x16x128 MFMAs (e4m3 operands, whole slabs; what 3 runs from K = 4096 on; these MFMAs
 * add 128 products per instruction instead of 64, so a sum can differ from the others' in its last fp32 bits); 6 and 8
 * are not assigned (CRL_ERR_ARG). 9 and 10 fall back to 7 where K is not whole slabs. 11 and 12 name the two
 * 128x128 kernels (same sums and bits as 2): 11 = fed by direct-to-LDS loads through a four-stage ring (whole slabs; what 2
 * runs for at most one tile per CU), 12 = register-staged (any K; 11 hands over to it where K is not whole slabs).
 * 15 and 16 = the 64x64 tile on an eight-stage and the 32x32 tile on a sixteen-stage ring of direct-to-LDS loads (same sums
 * and bits as 1; whole slabs; e4m3 operands with a 16-bit or e4m3 output, bf16/f16 operands with an output of their own
 * type, bf16 operands with an fp32 output; else CRL_ERR_ARG). Below 256 tiles of
 * 128x128, tile 0 runs 16 while every 32x32 tile has a CU of its own, 15 while every 64x64 tile has, 11 beyond, and 1 where
 * they do not apply.
 * 13 and 14 name the kernel for K = 256 e4m3 elements whose workgroups keep 256 rows of A in registers and walk N (the
 * attention-bias generator's product): a bare scaled product (no bias, activation, residual or amax; alpha = 1) into a
 * bf16/f16 output of more than 64 MB, M a multiple of 256, N of 128; anything else is CRL_ERR_ARG. 13 writes C row-major
 * (same result bits as 3); 14 writes it (ldc == N) in contiguous blocks of 256 rows x 128 columns, element (m, n) at
 * ((m / 256) * (N / 128) + n / 128) * 32768 + (m % 256) * 128 + n % 128, which is 1.6 times faster and what the model uses. */
int crl_gemm(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
             int M, int N, int K, int in_dtype, int out_dtype,
             const float* bias, int act, float descale, float alpha,
             const void* res, int64_t ldr, int res_dtype, float out_scale, float* amax,
             int tile, void* stream);
/* crl_gemm with its columns split over two outputs: columns [0, nsplit) go to C, columns [nsplit, N) to C2 (row stride
 * ldc2, column n at n - nsplit), both of out_dtype; epilogue descale * acc + bias. This is how the BT4-class layer runs the
 * q, k, v projections and the 32-column compression of the attention-bias generator as one product over one
 * concatenated weight (the reference's layers call one nn.Linear per projection, new_paradigm/attn.py:501-503; the
 * generator follows lc0's smolgen, which the reference does not contain). tile: 0 = automatic, or 3, 7, 10 as in crl_gemm
 * (same sums and result bits in every case). With e4m3 operands, a 16-bit output of more than 64 MB, M in whole 256-row
 * tiles, nsplit a multiple of 256 and at most 32 columns behind it, the 256x256 kernel's last tile column computes the
 * columns of C2 as well instead of a tile column of their own. */
int crl_gemm_split(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, void* C2, int64_t ldc2, int nsplit,
                   int M, int N, int K, int in_dtype, int out_dtype, const float* bias, float descale, int tile, void* stream);
/* No counterpart in the reference: crl_gemm with tile = 4 (K cut into slices, a second kernel adds them) for callers that
 * cannot allocate device memory, i.e. code under HIP graph capture, serving loops and harnesses that forbid hipMalloc.
 * The partial sums of the slices go to a fixed array of crl_gemm_static_scratch_bytes() = 8 MB inside the library's
 * device image (one copy per GPU, held until the process ends) instead of the per-stream workspace crl_gemm allocates on
 * first use; the call allocates and frees nothing. Arguments and result bits are those of crl_gemm(..., tile = 4, ...).
 * Products whose slices need more (slices * M * round_up(N, 8) * 4 bytes; slices <= 16) fail with CRL_ERR_ARG and a
 * message naming both sizes. Every call on a GPU uses that GPU's one array: calls that overlap in time on one GPU
 * (different streams or threads) race. Nothing in the array has to start at zero (each launch overwrites what it reads). */
int crl_gemm_static_scratch(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                            int M, int N, int K, int in_dtype, int out_dtype,
                            const float* bias, int act, float descale, float alpha,
                            const void* res, int64_t ldr, int res_dtype, float out_scale, float* amax, void* stream);
int64_t crl_gemm_static_scratch_bytes(void);
/* F.layer_norm(x,(C,),gamma,beta,eps) (model_bis.py:34). out (out_dtype) and/or out_fp8
 * (value*fp8_scale, e4m3) may be given. */
int crl_layernorm(const void* x, int64_t ldx, int in_dtype, const float* gamma, const float* beta,
                  void* out, int out_dtype, uint8_t* out_fp8, float fp8_scale, int64_t ldo,
                  int rows, int C, float eps, float* amax, void* stream);
/* RMSNorm, x / sqrt(mean(x^2) + eps) * gamma, with the same outputs as crl_layernorm. The reference's models use
 * LayerNorm only (model_bis.py:25-34, new_paradigm/value.py:36-37); this is the norm crl_model_config.norm_rms selects. */
int crl_rmsnorm(const void* x, int64_t ldx, int in_dtype, const float* gamma, void* out, int out_dtype, uint8_t* out_fp8,
                float fp8_scale, int64_t ldo, int rows, int C, float eps, float* amax, void* stream);
/* Attention over 64 tokens per position, q/k/v of in_dtype (bf16 or f16) with head h at columns [h*head_dim, ...).
 * mode CAUSAL: model_bis.py:71; RELSHIFT: new_paradigm/attn.py:507-521 with pos = pos_proj(PE)
 * (in_dtype [64,H*head_dim]) and u_bias/v_bias fp32[H*head_dim]; BIAS: bias of in_dtype [B,H,64,64] in the
 * order crl_attn_bias_slot defines. out is of in_dtype or fp8 (value*out_scale) [B*64, ldo]. */
int crl_attention(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v, int64_t ldv, int in_dtype,
                  void* out, int64_t ldo, int out_dtype, float out_scale,
                  int B, int H, int head_dim, int mode, float scale,
                  const void* bias, const void* pos, const float* u_bias, const float* v_bias,
                  float* amax, void* stream);
int crl_attn_bias_slot(int query, int key);
/* logits + (1-mask)*(-999); softmax(./T); T==0 -> one-hot arg-max (model_bis.py:382-392).
 * logits f32 [B,V] (ldl), mask uint8 [B,V] or NULL, probs f32 [B,V] or NULL, argmax int32[B] or NULL. */
int crl_masked_softmax(const float* logits, int64_t ldl, const uint8_t* mask, int64_t ldm,
                       float* probs, int64_t ldp, int32_t* argmax, int B, int V, float temperature, void* stream);
/* Leela/compare_policy.py:493-523 map_leela_to_rl on device: src f32 [B,1858] -> dst f32 [B,1929];
 * white_to_move uint8[B] selects identity or the rank-mirrored slot. */
int crl_leela_to_rl(const float* src, int64_t lds, float* dst, int64_t ldd, const uint8_t* white_to_move, int B, void* stream);

/* ------------------------------------------------------------------ device: models */
typedef struct crl_model crl_model;

typedef struct crl_model_config {
  int32_t arch;           /* CRL_ARCH_* */
  int32_t n_layer;
  int32_t d_model;
  int32_t n_head;
  int32_t d_ff;
  int32_t fp8;            /* 1: trunk linears (qkv, out-proj, ffn) run in e4m3 with static per-tensor scales */
  int32_t micro_batch;    /* positions per pass through the trunk; 0 = default */
  int32_t stream_f32;     /* residual stream (the tensors the residual additions and the norms read) in fp32 instead of
                             the 16-bit type: 0 = default (fp32 for GPT64, 16-bit for BT4 and BT4-class), 1 = fp32,
                             -1 = 16-bit. The GEMM operands stay 16-bit / e4m3 either way. */
  int32_t head_dtype;     /* CRL_BF16 or CRL_F16: element type of the policy/value head GEMM inputs; 0 = act_dtype */
  int32_t smolgen_compress, smolgen_hidden, smolgen_gen;  /* BT4-class; 0 = 32/256/256 */
  float eps;              /* LayerNorm epsilon; 0 = 1e-5 */
  int32_t act_dtype;      /* CRL_BF16 (default) or CRL_F16: 16-bit element type of activations and weights */
  int32_t ln_fold;        /* e4m3 BT4-class with a 16-bit bf16 stream: the trunk norms write only their e4m3 copy and row
                             statistics, and the product that takes the normalised tensor as its residual normalises it
                             in its epilogue. 0 = default (on), -1 = off (every norm writes its 16-bit output). */
  int32_t norm_rms;       /* 1: the norms of the trunk (and GPT64's ln_f) are RMSNorm, x/sqrt(mean(x^2)+eps)*weight; their
                             .bias entries are accepted and ignored. 0 = LayerNorm as in the reference. */
  int32_t fp8_lm_head;    /* fp8 models: the output heads run in e4m3 as well, as the reference's recipe quantises every
                             nn.Linear (model_fp8.py:43,45,90,92,140): lm_head for GPT64; policy_tokens_lin, queries_pol|keys_pol
                             and value_head.dense1 for BT4-class. 1 = e4m3 heads, -1 = 16-bit heads, 0 = default: on for GPT64
                             (the reference's fp8 model), off for BT4-class (whose policy is a product of two quantised
                             projections: its error against fp32 grows by half for under two percent of the pass). */
} crl_model_config;

/* GPT(config) / BT4(...) constructors (model_bis.py:127-157, new_paradigm/value.py:122-152). */
int crl_model_create(const crl_model_config* cfg, crl_model** out);
void crl_model_destroy(crl_model* m);
/* load_state_dict(): hand over one tensor by its state-dict key as host fp32 (the library
 * keeps its own converted copy). Keys are listed by crl_model_expected_key(). */
int crl_model_set_weight(crl_model* m, const char* key, const float* data, int64_t numel);
/* i-th expected state-dict key and its element count; NULL when i is out of range. */
const char* crl_model_expected_key(crl_model* m, int i, int64_t* numel);
/* Convert/pack weights to device (bf16, fp8 and re-ordered copies). Needs a GPU. */
int crl_model_finalize(crl_model* m);
/* fp8 only: run the bf16 path on calibration positions and derive the static activation
 * scales 448/amax (pretrain_fp8.py:75-79 uses DelayedScaling amax history; here the history
 * is one calibration batch). Synchronises the stream. */
int crl_model_calibrate(crl_model* m, const float* planes, int B, void* stream);
/* Read / overwrite the activation amax table, float[n_layer*5]: per layer the input of q|k|v, the attention output,
 * the inputs of the two FFN linears and the input of the shared attention-bias generator (BT4-class only, else 0).
 * With n = (n_layer+1)*5 the table carries one more row for the e4m3 head linears: its first entry is the amax of lm_head's
 * input (GPT64; taken by crl_model_calibrate over every token of ln_f) or of the trunk output that policy_tokens_lin and
 * value_head.dense1 read (BT4-class), its second entry the amax of the policy tokens that queries_pol|keys_pol read
 * (BT4-class). While the entries a model needs are 0 (never calibrated, or only the short table was set) its heads run on
 * their 16-bit copies. */
int crl_model_get_amax(crl_model* m, float* out, int n);
int crl_model_set_amax(crl_model* m, const float* in, int n);
/* The forward pass. planes: device f32 [B,64,19] (GPT.forward batch[0] / BT4.forward inp[0]).
 * policy_logits: device f32 [B, vocab] with vocab = 1929 (GPT64: logits of token 63,
 * model_bis.py:370; BT4: value.py:187) or 1858 (BT4-class). wdl_logits: device f32 [B,3]
 * in the order [black win, draw, white win] (value.py:248), NULL for GPT64 or to skip.
 * B = 0 is accepted by this and the two entry points below: nothing is launched or written. */
int crl_model_forward(crl_model* m, const float* planes, int B, float* policy_logits, float* wdl_logits, void* stream);
/* Same from the compact board form (device uint8[B,64] ids + uint8[B,4] flags). */
int crl_model_forward_compact(crl_model* m, const uint8_t* ids, const uint8_t* flags, int B,
                              float* policy_logits, float* wdl_logits, void* stream);
/* CRL_ARCH_GPT64 with move tokens: GPT.forward((planes, idx), compute_loss) of model_bis.py:171-199. idx [B,t] int64 are
 * the t move tokens that follow the 64 board tokens (embedded with the tied lm_head weight plus rows 64.. of `pe`,
 * 64+t <= rows of `pe` given to crl_model_set_weight). last_logits [B,1929] receives the logits of the last token
 * (compute_loss=False, :195-196), all_logits [B,64+t,1929] those of every token (compute_loss=True, :191); either
 * may be NULL. Attention is causal over all 64+t tokens. */
int crl_model_forward_tokens(crl_model* m, const float* planes, const int64_t* idx, int B, int t, float* last_logits,
                             float* all_logits, void* stream);
/* Sequence generation for CRL_ARCH_GPT64 with cached keys and values: GPT.generate_sequence (rules = 1,
 * model_bis.py:213-263) and GPT.generate_sequence_raw (rules = 0, :266-311). sequences [B, steps+1] int64 receives
 * <thinking> (1924) followed by `steps` tokens: arg-max for temperature 0, else one draw from softmax(logits/temperature)
 * (inverse CDF with a counter-based generator keyed by seed, sequence and step: reproducible, not torch's stream).
 * With rules the forced tokens of :252-259 apply: after five end_variation tokens the next is </thinking>, and the
 * token two places after a </thinking> is end. step_out [B, steps, 1929] (optional) receives every step's
 * probabilities, or its logits when out_logits != 0 (return_logits of :266). The 65-token prefix is run once; every
 * later token costs one row per sequence against the cache (the reference re-runs the whole prefix per token).
 * steps <= rows(pe) - 64 and <= 960; B*65 tokens must fit one micro-batch. Runs in the 16-bit type also for fp8 models.
 * crl_model_set_decode_graph(m, 1) records the per-token launches once into a HIP graph (from the second token on;
 * the kernels then read the token index from a device counter) and replays it; results are bit-identical, the call
 * returns after the stream has drained, and the stream must not itself be under capture. It is off by default: a
 * token step is bound by its kernels' run time on the device, not by the host's launches (measured: no gain at 128
 * sequences), so the option is for hosts that cannot keep up. The profiling mode always launches plainly. */
int crl_model_generate(crl_model* m, const float* planes, int B, int steps, float temperature, uint64_t seed, int rules,
                       int64_t* sequences, float* step_out, int out_logits, void* stream);
int crl_model_set_decode_graph(crl_model* m, int on);
/* Host front-end of leaf evaluation: n FEN strings in host memory -> results in host memory. Replaces the per-FEN
 * Python of model_bis.py:358-398 and new_paradigm/value.py:214-243,275-317 (encode_fens, the legal-move loop with
 * policy_index.index per move, mask, softmax/arg-max) for whole batches. The positions are walked in chunks of
 * `chunk`: host threads parse, encode (64 piece ids + 4 flag bytes) and build the legal mask of chunk i+1 into
 * pinned memory while the device runs chunk i; uploads go over a copy stream of their own. probs [n, V] receives
 * softmax((logits + (1-mask)*-999)/temperature) (one-hot at the arg-max for temperature 0), wdl [n,3] the value
 * logits, best [n] the index of the best legal move; each may be NULL. V and the move order are those of the model
 * (1929 / crl_policy_index, or 1858 side-to-move-frame / crl_policy_leela for CRL_ARCH_BT4CLASS). One call at a time
 * per model; the staging buffers (2 chunks, pinned + device) stay with the model until it is destroyed. The call runs
 * on streams of its own: it first waits for everything queued on the device (hipDeviceSynchronize), so forwards issued
 * earlier on any stream of this model are complete before it touches the model's workspace, and it returns with its own
 * work finished. crl_model_search_1ply behaves the same way. */
int crl_model_evaluate_fens(crl_model* m, const char* const* fens, int n, int chunk, float temperature, float* probs,
                            float* wdl, int32_t* best, int threads);
/* Batched 1-ply value search: BT4.calculate_move_values / get_best_move_value (new_paradigm/value.py:319-400) for n root
 * positions at once. Every legal move of every root is made on the host, all child positions go through the same
 * chunked pipeline as crl_model_evaluate_fens (value head only: no masks, no policy download), and per root the value
 * of a child for the side to move at the root is 0.5*P(draw) + P(win for that side) with P = softmax of the child's
 * [black win, draw, white win] logits (:343-352). best_uci6 [n,6] receives the move with the largest value
 * (temperature 0) or one draw from softmax(values/temperature) (:384-394; inverse CDF with a generator keyed by seed and
 * root index, not torch's stream); a root without legal moves gets an empty string (the reference raises there).
 * Optional: n_moves [n]; moves_uci6 [total,6] and values [total], the children of root i at
 * sum(n_moves[0..i)) onwards in move-generation order, total <= capacity or the call fails. Not for CRL_ARCH_GPT64. */
int crl_model_search_1ply(crl_model* m, const char* const* fens, int n, int chunk, float temperature, uint64_t seed,
                          char* best_uci6, int32_t* n_moves, char* moves_uci6, float* values, int64_t capacity, int threads);
/* Verification hooks with no counterpart in the reference (its layers are nn.Modules one can call one at a time:
 * new_paradigm/value.py:58-75 EncoderLayer.forward, model_bis.py:110-113 Block.forward). crl_model_run_layers (CRL_ARCH_BT4CLASS
 * only) runs encoder layers [first, last) on a caller-supplied layer input x_in (device f32 [B*64, d_model], at most one micro-batch) and
 * writes the output of layer last-1 to x_out (device f32, same shape). The window's first layer treats x_in as layer 0
 * treats the embedding (stored in the model's activation type; for an fp8 model its e4m3 copy is quantised from x_in
 * directly with that layer's scale), its last layer writes its output in the 16-bit type as the trunk's last layer does,
 * the layers between run exactly as inside crl_model_forward. A parity test can so hand every layer the oracle's own
 * input and hold its output to a per-layer bar. crl_model_read_tensor copies one of the workspace tensors the last call
 * left behind to `out` (device): "x8", "h8", "ao8" (e4m3 [tokens, d_model]: the inputs of q|k|v, of FFN-1 and of the
 * out-projection), "f8" (e4m3 [tokens, d_ff]: the input of FFN-2), "t" (the un-normalised residual sum in the stream's
 * type); only the e4m3 copies an fp8 model writes are meaningful. */
int crl_model_run_layers(crl_model* m, const float* x_in, int B, int first, int last, float* x_out, void* stream);
int crl_model_read_tensor(crl_model* m, const char* name, void* out, int64_t bytes, void* stream);
int crl_model_vocab(const crl_model* m);
/* 2*MAC count of one position through this model (for roofline accounting). */
double crl_model_flops_per_position(const crl_model* m);
/* Switch: bracket every kernel launch with HIP events on the call's stream; each forward then
 * ends with a stream synchronise and accumulates, per kernel family, the elapsed milliseconds,
 * the launch count and (GEMMs) the 2*M*N*K work. Families: 0 fp8 GEMM, 1 attention,
 * 2 LayerNorm, 3 embedding, 4 policy QK^T, 5 16-bit GEMM. flops6 may be NULL. */
int crl_model_set_profiling(crl_model* m, int on);
int crl_model_get_profile(crl_model* m, double* ms6, int64_t* launches6, double* flops6);

/* Causal attention over T tokens per position (any T in 1..4096): F.scaled_dot_product_attention(q,k,v,is_causal=True)
 * of model_bis.py:71 for the 64+t token sequences of model_bis.py:171-199. Layout and types as crl_attention; rows of
 * position b are b*T .. b*T+T-1. */
int crl_attention_causal(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v, int64_t ldv, int in_dtype, void* out,
                         int64_t ldo, int out_dtype, float out_scale, int B, int H, int head_dim, int T, float scale, float* amax, void* stream);
/* One token per row of logits [B, V] (V <= 2048): arg-max (lowest index among equals) for temperature 0, else one
 * draw from softmax(logits/temperature), i.e. torch.argmax / F.softmax + torch.multinomial of model_bis.py:242-247,
 * 385-392. The draw is the inverse CDF at a uniform number that depends only on (seed, row, step). probs [B, V]
 * (optional) receives the softmax. */
int crl_sample(const float* logits, int64_t ldl, int B, int V, float temperature, uint64_t seed, int step, int64_t* tokens, float* probs,
               void* stream);
/* Per-row log-softmax statistics of logits [rows, V] (V <= 2048), each output optional:
 *   logp[r]     = log_softmax(logits[r])[target[r]]      (0 where target[r] == ignore_index or outside 0..V-1)
 *   ref_logp[r] = log_softmax(ref_logits[r])[target[r]]
 *   kl[r]       = sum_v softmax(logits[r])[v] * (log_softmax(logits[r])[v] - log_softmax(ref_logits[r])[v])
 * i.e. the terms of F.cross_entropy in model_bis.py:192-193 and of the GRPO scoring of grpo_refactored.py:337-342
 * (new_log_probs, ref_log_probs, per_token_kl and their gather at the sampled tokens). */
int crl_token_scores(const float* logits, int64_t ldl, const float* ref_logits, int64_t ldr, const int64_t* target, int rows, int V,
                     int64_t ignore_index, float* logp, float* ref_logp, float* kl, void* stream);
/* out[0] = mean of -logp[r] over rows with target[r] != ignore_index (F.cross_entropy(..., ignore_index), model_bis.py:193);
 * summed in a fixed order; 0 when no row counts. */
int crl_masked_nll_mean(const float* logp, const int64_t* target, int64_t ignore_index, int rows, float* out, void* stream);

/* Measurement probe with no counterpart in the reference: every CU runs 8 waves that issue
 * 32x32 MFMAs back to back from registers (dtype CRL_BF16, CRL_F16 or CRL_FP8; iters rounds of 8
 * MFMAs per wave). random_bits = 0 uses all-zero operands (clock-limited peak), 1 uses random
 * operand bits (the rate the part sustains under its power limit). Returns the sustained
 * TFLOP/s and the shader clock in GHz the kernel ran at. Synchronises the stream. */
int crl_probe_mfma(int dtype, int random_bits, int iters, double* tflops, double* ghz, void* stream);

/* Measurement probe with no counterpart in the reference: would the memory-bound kernels of a pass overlap with its
 * products if the two ran on disjoint sets of CUs? Two streams with CU masks (gemm_cus of the 256 CUs for the e4m3
 * product rows x 1024 x 1024, the rest for the trunk LayerNorm over `rows` rows of 1024) are timed alone on all CUs, alone on
 * their share and side by side. out8: product us/launch on all CUs, on its share, beside the norm; norm us/launch on all
 * CUs, on its share, beside the product; wall time of the side-by-side run in ms; the same launches back to back on all
 * CUs in ms. gemm_cus = 256 uses two plain streams instead (both kernels may use every CU); tile is the crl_gemm tile code of
 * the product (0 = the library's choice). Allocates its own operands; synchronises the device. */
int crl_probe_cu_split(int gemm_cus, int tile, int rows, int iters, double* out8);

#ifdef __cplusplus
}
#endif
#endif /* CHESSRL_AMD_H */
