/*
 * CPU ORACLE - TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C restatement of the reference's algorithms for the quantized
 * decode path (CAI Neural API, Free Pascal).  Only tests, the smoke check
 * and the benchmark's cpu_baseline leg may load this library; the shipped
 * library (libcaihip.so) never links or calls it.
 *
 * Every function cites the reference file:line (relative to the reference
 * checkout root) whose arithmetic it follows.
 */
#ifndef CAI_ORACLE_H
#define CAI_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml tensor type ids: neural/neuralgguf.pas:86-98 */
enum {
  ORC_F32 = 0, ORC_F16 = 1, ORC_Q4_0 = 2, ORC_Q4_1 = 3, ORC_Q5_0 = 6, ORC_Q5_1 = 7, ORC_Q8_0 = 8, ORC_Q2_K = 10, ORC_Q3_K = 11,
  ORC_Q4_K = 12, ORC_Q5_K = 13, ORC_Q6_K = 14,
  ORC_I8ROW = 100 /* per-row symmetric int8 (neural/neuralvolume.pas:926-987) */
};

/* ---- scalar codecs ---- */
float    orc_f16_to_f32(uint16_t bits);             /* neuralsafetensors.pas:294-329 */
uint16_t orc_f32_to_f16(float v);                   /* neuralsafetensors.pas:338-396 */
void     orc_q4k_scale_min(const uint8_t* packed12, uint8_t* sc8, uint8_t* mn8); /* neuralgguf.pas:448-464 */

/* ---- block geometry ---- */
int64_t  orc_block_elems(int type);
int64_t  orc_block_bytes(int type);
int64_t  orc_row_bytes(int type, int64_t cols);     /* -1 if cols is not a whole number of blocks */

/* ---- dequantizers: raw blocks -> fp32, n_elems must be whole blocks ---- */
void orc_dequant_q8_0(const uint8_t* raw, int64_t n_blocks, float* out);  /* neuralgguf.pas:1487-1503 + neuralvolume.pas:12564-12582 */
void orc_dequant_q4_0(const uint8_t* raw, int64_t n_blocks, float* out);  /* neuralgguf.pas:811-845 */
void orc_dequant_q4_k(const uint8_t* raw, int64_t n_blocks, float* out);  /* neuralgguf.pas:472-514 */
void orc_dequant_q6_k(const uint8_t* raw, int64_t n_blocks, float* out);    /* neuralgguf.pas:639-717 (DequantizeQ6K) */
void orc_quant_q6_k(const float* x, int64_t n_elems, uint8_t* out);        /* this build's packer; layout neuralgguf.pas:639-650 */
int  orc_dequant(int type, const void* raw, int64_t n_elems, float* out); /* neuralgguf.pas:1471-1523 */

/* ---- quantizers (make synthetic weights; only Q8_0 exists in the reference) ---- */
void orc_quant_q8_0(const float* x, int64_t n_elems, uint8_t* out);       /* neuralgguf.pas:1966-1989 */
void orc_quant_q4_0(const float* x, int64_t n_elems, uint8_t* out);       /* ggml quantize_row_q4_0_ref behaviour */
void orc_quant_q4_k(const float* x, int64_t n_elems, uint8_t* out);       /* affine fit; layout neuralgguf.pas:440-514 */
/* per-row symmetric int8: neuralvolume.pas:12501-12562 (scalar twin) */
void orc_quant_int8_row(const float* x, int64_t n, int8_t* codes, float* scale);

/* ---- row permutations ---- */
int64_t orc_gguf_deinterleaved_src_row(int64_t hf_row, int head_dim);     /* neuralgguf.pas:428-438 */
int64_t orc_map_target_neuron(int64_t row, int head_dim);                 /* neuralpretrained.pas:14792-14812 */

/* ---- linear layer:  y[b*rows+a] = act(dot(W[a], x[b]) (+bias[a])) ----
 * act: 0 none, 1 ReLU, 2 sigmoid, 3 tanh (neural.cl:114-146).
 * acc64 != 0 accumulates in double and rounds once (error-budget variant).
 * For ORC_I8ROW `raw` is int8 codes row-major and `scales` holds one float per row
 * (y = scale*sum(code*x) + bias, neuralvolume.pas:12693-12745). */
int orc_gemv(int type, const void* raw, const float* scales, int64_t rows, int64_t cols,
             const float* x, int n_b, const float* bias, int act, int acc64, float* y);

/* ---- elementwise layer math ---- */
void orc_rmsnorm(const float* x, const float* gain, int n, float eps, float* y);     /* neural.cl:1047-1085 */
void orc_rope_thetas(float base, int head_dim, float* theta_half);                   /* neural.cl:1510-1515 (host table) */
int  orc_rope_thetas_scaled(float base, int head_dim, int mode, float factor, int original_ctx, float low_freq_factor, float high_freq_factor, float* theta_half); /* neuralpretrained.pas:633-668 */
void orc_rope_interleaved(float* x, int n_heads, int head_dim, int pos, const float* theta_half); /* neural.cl:1517-1542 */
void orc_swiglu(const float* up_gate, int half, float* y);                           /* neural.cl:1213-1263 flag 1 */
void orc_softmax(const float* x, int n, float* y);                                   /* neural.cl:1594-1647 */
void orc_topk_gate(const float* probs, int n, int k, int renorm, float* gates_out, int* idx_out); /* tests/TestNeuralNumerical.pas:74997-75042 */
int  orc_argmax(const float* x, int n);                                              /* neuralchatengine.pas:683-697 */

/* ---- distribution pipeline ahead of the samplers (neuralchatengine.pas:1374-1396, 1495-1501) ----
 * softmax -> history penalty -> temperature, then the m most probable tokens, descending (ties: lower id first).
 * hist_ids are the DISTINCT tokens of the context with their occurrence counts.  Returns min(m, n). */
int orc_sample_candidates(const float* logits, int n, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                          float repetition, float frequency, float presence, float temperature, int m,
                          int32_t* tok_out, float* p_out);

/* ---- cached GQA decode attention, fp32, head-major cache (neural.cl:2354-2499) ----
 * k_cache/v_cache: [kv_heads][max_ctx][head_dim]; qkv row = [Q | K | V]. Appends at slot
 * cache_len, then attends over [j_start .. cache_len] where window>0 limits the range.
 * kv_f16 == 1 rounds the appended K,V through IEEE half first (fp16 cache model). */
void orc_attn_decode(const float* qkv, int q_heads, int kv_heads, int head_dim,
                     float* k_cache, float* v_cache, int max_ctx, int cache_len,
                     int window, float softcap, int kv_f16, float* out);

/* The same under sink + recent-window eviction (neuraldecode.pas:1257-1276); the caches stay unbounded (max_ctx rows
 * must cover the whole stream), rows outside [0, sinks) u [len - recent, len) are masked once len > sinks + recent. */
void orc_attn_decode_evict(const float* qkv, int q_heads, int kv_heads, int head_dim,
                           float* k_cache, float* v_cache, int max_ctx, int cache_len,
                           int sinks, int recent, float softcap, int kv_f16, float* out);

/* ---- int8 KV cache: per-row symmetric codes + fp32 scale (neural.cl:2501-2687) ----
 * codes [kv_heads][max_ctx][head_dim], scales [kv_heads][max_ctx]. */
float orc_max_abs_finite(const float* x, int n);                                     /* neuralvolume.pas:12471 */
void orc_kv_quant_row(const float* x, int n, int8_t* codes, float* scale);           /* neural.cl:2549-2578 */
void orc_attn_decode_i8(const float* qkv, int q_heads, int kv_heads, int head_dim,
                        int8_t* k_codes, float* k_scales, int8_t* v_codes, float* v_scales,
                        int max_ctx, int cache_len, int window, float softcap, float* out);

/* ---- whole decoder (Llama / Qwen2 / OLMoE families), one token at a time ---- */
typedef struct orc_model orc_model;

typedef struct {
  int32_t n_layers, d_model, n_q_heads, n_kv_heads, head_dim, ffn, vocab, max_ctx;
  float   eps, rope_theta;
  int32_t window;         /* sliding window (0 = none) */
  int32_t qk_norm_full;   /* OLMoE: RMSNorm over full q / k width before RoPE */
  int32_t n_experts, top_k, norm_topk; /* n_experts == 0 -> dense SwiGLU FFN */
  int32_t kv_f16;         /* cache element model: 0 fp32, 1 rounded to half, 2 int8 codes + row scale */
  int32_t acc64;          /* accumulate linear layers in double */
  int32_t evict_sinks, evict_recent; /* sink + recent-window eviction (0, 0 = off); max_ctx must still cover the stream */
} orc_config;

/* tensor slots */
enum {
  ORC_W_EMBED = 0, ORC_W_HEAD = 1,                      /* layer = -1 */
  ORC_W_Q = 2, ORC_W_K = 3, ORC_W_V = 4, ORC_W_O = 5,
  ORC_W_GATEUP = 6,  /* rows 0..I-1 = up, I..2I-1 = gate (neuralpretrained.pas:240-243); MoE: bank, expert e rows e*2I.. */
  ORC_W_DOWN = 7,    /* MoE: bank, expert e rows e*H.. */
  ORC_W_ROUTER = 8
};
/* vector slots */
enum { ORC_V_ATTN_NORM = 0, ORC_V_MLP_NORM = 1, ORC_V_FINAL_NORM = 2, ORC_V_Q_NORM = 3, ORC_V_K_NORM = 4 };

orc_model* orc_model_new(const orc_config* cfg);
void orc_model_free(orc_model* m);
/* The model keeps the pointers; the caller keeps the memory alive. */
int  orc_model_set_tensor(orc_model* m, int layer, int slot, int type, int64_t rows, int64_t cols,
                          const void* raw, const float* scales, const float* bias);
int  orc_model_set_vec(orc_model* m, int layer, int slot, const float* v, int n);
void orc_model_set_thetas(orc_model* m, const float* theta_half, int n);
void orc_model_set_rope_out_scale(orc_model* m, float s);
float orc_rope_out_scale(int mode, float factor);
void orc_model_reset(orc_model* m);
void orc_model_truncate(orc_model* m, int n);
int  orc_model_len(const orc_model* m);
/* Runs one token at position `pos` (== current cache length). logits may be NULL. Returns argmax. */
int  orc_model_step(orc_model* m, int token, int pos, float* logits);

/* The input of the vocabulary projection at the last step (final RMSNorm of the residual stream, d_model floats): HiddenState of
 * the reference session (neural/neuraldecode.pas:5850-5857 with the heuristic of 6794-6807: the layer feeding the head). */
const float* orc_model_hidden(const orc_model* m);
void orc_model_swap_selection(orc_model* m, int layer, int pos);       /* test hook: rank k and k + 1 trade places there */
const float* orc_model_router_probs(const orc_model* m, int layer);   /* block `layer`'s router soft-max at the last step */
/* PromptLookupDraft on token ids (neural/neuraldecode.pas:7742-7765): the (at most num_draft) tokens that followed the most
 * recent STRICTLY EARLIER occurrence of the context's last match_len tokens.  Returns the draft length. */
int  orc_prompt_lookup_draft(const int32_t* ctx, int n_ctx, int match_len, int num_draft, int32_t* draft);

#ifdef __cplusplus
}
#endif
#endif
