/*
 * caihip - C ABI of the MI355X (gfx950) quantized LLM decode path for CAI Neural API.
 *
 * Plain C, cdecl, opaque handles, int error codes, no exceptions across the boundary.
 * The library owns all device memory; every create has a destroy; host pointers are never
 * retained after a call returns.  All calls enqueue on one in-order HIP stream owned by the
 * library (the analogue of the reference's single shared in-order OpenCL queue,
 * examples/ChatTerminal/README.md:174-180).  Calls from several host threads are serialised by one
 * lock inside the library; cai_last_error reports the calling thread's own last failure.
 *
 * Citations are file:line in the reference checkout (joaopauloschuler/neural-api).
 */
#ifndef CAIHIP_H
#define CAIHIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes ---- */
#define CAI_OK               0
#define CAI_ERR_INVALID     (-1)  /* bad argument / shape */
#define CAI_ERR_HIP         (-2)  /* HIP runtime error (text in cai_last_error) */
#define CAI_ERR_NOMEM       (-3)
#define CAI_ERR_UNSUPPORTED (-4)
#define CAI_ERR_STATE       (-5)  /* not initialised, slot not set, cache full ... */

/* ---- weight storage types: ggml ids (neural/neuralgguf.pas:86-98) ---- */
#define CAI_F32    0
#define CAI_F16    1
#define CAI_Q4_0   2
#define CAI_Q4_1   3   /* the six types below stay resident as the stored block stream (neural/neuralgguf.pas:516-648, 718-944) */
#define CAI_Q5_0   6
#define CAI_Q5_1   7
#define CAI_Q8_0   8
#define CAI_Q2_K   10
#define CAI_Q3_K   11
#define CAI_Q4_K   12
#define CAI_Q5_K   13
#define CAI_Q6_K   14  /* 210-byte super-blocks (neural/neuralgguf.pas:639-717); resident as aligned ql|qh records + planes of scales and d */
#define CAI_I8ROW  100  /* per-row symmetric int8 + fp32 row scale (neural/neuralvolume.pas:926-987) */

/* ---- activation opcodes fused into the linear layer (neural/neural.cl:114-146) ---- */
#define CAI_ACT_NONE    0
#define CAI_ACT_RELU    1
#define CAI_ACT_SIGMOID 2
#define CAI_ACT_TANH    3

/* ---- pointer-space flags for compute calls ---- */
#define CAI_X_DEVICE 1  /* input pointer is device memory (a producer's resident buffer; cf. pExternalVBs, neural/neuralopencl.pas:946) */
#define CAI_Y_DEVICE 2  /* output pointer is device memory (no read-back; cf. ResultBuffer, neural/neuralopencl.pas:383-388) */
#define CAI_MATRIX_CORES 4  /* cai_qgemm only: take the matrix-core kernels even for a matrix small enough that the dispatcher would keep it on the vector units */

/* ---- KV cache element types ---- */
#define CAI_KV_F32 0
#define CAI_KV_F16 1
#define CAI_KV_I8  2  /* codes in [-127,127] + one fp32 scale per cached row (scale = max|row|/127), the format of
                         cai_sdpa_append_kv_int8 / QuantizeCacheRow, neural/neural.cl:2501-2580 */

typedef struct cai_qw_s*      cai_qw_t;       /* resident quantized weight matrix */
typedef struct cai_kv_s*      cai_kv_t;       /* KV cache of one sequence, all layers */
typedef struct cai_kv_snap_s* cai_kv_snap_t;  /* deep copy of a KV cache's live rows */
typedef struct cai_decoder_s* cai_decoder_t;  /* step-resident decoder */

/* =====================================================================================
 * Library lifetime.  Replaces TNNet.EnableOpenCL(PlatformId, DeviceId, shared)
 * (neural/neuralchatengine.pas:1156-1157): selects the GPU and creates the stream.
 * ===================================================================================== */
int cai_init(int device_ordinal);
int cai_shutdown(void);
/* Copies the text of the last error of the calling process into buf (NUL terminated). */
int cai_last_error(char* buf, int buf_len);
int cai_device_name(char* buf, int buf_len);
/* Blocks until all enqueued work is finished (FinishAndLoadResult's clFinish, neural/neuralopencl.pas:1058-1104). */
int cai_sync(void);
/* hipStream_t of the library, for callers that record their own events. */
int cai_get_stream(void** stream_out);
/* HIP-event stopwatch on the library stream: start, enqueue work, stop -> elapsed ms. */
int cai_timer_start(void);
int cai_timer_stop(float* ms_out);

/* Device buffers for resident activations. */
int cai_dev_alloc(int64_t bytes, void** ptr_out);
int cai_dev_free(void* ptr);
int cai_dev_upload(void* dst_dev, const void* src_host, int64_t bytes);
int cai_dev_download(void* dst_host, const void* src_dev, int64_t bytes);
/* Plain device-to-device copy kernel (16-byte loads/stores; bytes must be a multiple of 16).  Also the known-size
 * reference against which hardware traffic counters are scaled. */
int cai_dev_copy(void* dst_dev, const void* src_dev, int64_t bytes);

/* =====================================================================================
 * Resident quantized weights.
 * Replaces TDotProductSharedKernel.PrepareForComputeInt8(pCodes, pScales, NumAs, pSize, VBs)
 * (neural/neuralopencl.pas:844-891): a blocking one-time upload; staging may be freed on return.
 * `blocks` holds `rows` rows of cols/block_elems GGUF blocks, row-major [out][in], exactly the
 * bytes of a GGUF tensor (neural/neuralgguf.pas:100-138, 226-236).  It may be a host or a device
 * pointer.  `bias` (rows floats, host) may be NULL.
 * ===================================================================================== */
int cai_qw_create(int qtype, int64_t rows, int64_t cols, const void* blocks, const float* bias, cai_qw_t* out);
/* Per-row int8 form: codes row-major [rows][cols], one fp32 scale per row
 * (TNNetVolume.QuantizeInt8 output, neural/neuralvolume.pas:12501-12562). */
int cai_qw_create_int8row(int64_t rows, int64_t cols, const int8_t* codes, const float* scales,
                          const float* bias, cai_qw_t* out);
int cai_qw_destroy(cai_qw_t w);                       /* UnprepareForCompute, neural/neuralopencl.pas:527-562 */
int cai_qw_info(cai_qw_t w, int* qtype, int64_t* rows, int64_t* cols, int64_t* device_bytes);
/* Dequantizes rows [row0, row0+n_rows) on the device into fp32 (bit-exact to DecodeGGMLSpan,
 * neural/neuralgguf.pas:1471-1523).  flags: CAI_Y_DEVICE. */
int cai_qw_dequant_rows(cai_qw_t w, int64_t row0, int64_t n_rows, float* out, int flags);

/* =====================================================================================
 * Linear layer forward (TNNetPointwiseConvLinear / TNNetFullConnectLinear).
 * Replaces ComputeInt8 + FinishAndLoadResult (neural/neuralopencl.pas:946-1104):
 *   y[b*rows + a] = act( dot(W[a], x[b*cols ..]) + bias[a] ),  b < n_b  (1 <= n_b <= 8)
 * Weights are dequantized in registers; accumulation is fp32.
 * ===================================================================================== */
int cai_qgemv(cai_qw_t w, const float* x, int n_b, float* y, int act, int flags);
/* Fused feed-forward front half: TokenRMSNorm(gain, eps) -> gate|up projection -> SwiGLU in one kernel
 * (TNNetTokenRMSNorm + TNNetPointwiseConvLinear(2I) + TNNetSwiGLU, neural/neuralpretrained.pas:16815-16862;
 * row layout up = rows 0..I-1, gate = rows I..2I-1, neural/neuralpretrained.pas:240-243).
 *   y[b*I + i] = up_i(h_b) * silu(gate_i(h_b)),  h_b = rmsnorm(x_b) (gain == NULL: h_b = x_b)
 * `gain` lives where x lives (host, or device with CAI_X_DEVICE).  Block-quantized weights only. */
int cai_ffn_gateup(cai_qw_t gateup, const float* x, const float* gain, float eps, int n_b, float* y, int flags);
/* Multi-token form on the matrix cores (prefill): x is [n_tokens][cols], y is [n_tokens][rows].
 * No counterpart in the reference, whose prefill is token-at-a-time
 * (neural/neuralchatengine.pas:1466-1470); results equal n_tokens GEMVs to about 1e-6 relative (exact integer weight
 * operands, activations carried as two f16 = 22 significant bits).  flags: CAI_X_DEVICE | CAI_Y_DEVICE | CAI_MATRIX_CORES. */
int cai_qgemm(cai_qw_t w, const float* x, int n_tokens, float* y, int flags);

/* =====================================================================================
 * Elementwise layer math on fp32 rows.  flags: CAI_X_DEVICE | CAI_Y_DEVICE.
 * ===================================================================================== */
/* TNNetTokenRMSNorm (neural/neural.cl:1047-1085, FUseMean = 0); x, y: [n_tokens][n]. */
int cai_rmsnorm(const float* x, const float* gain_host, int n, int n_tokens, float eps, float* y, int flags);
/* TNNetRotaryEmbedding, interleaved pairs, head-tiled theta (neural/neural.cl:1517-1542);
 * in place over x = [n_heads][head_dim] at absolute position pos. */
int cai_rope(float* x, int n_heads, int head_dim, int pos, float theta_base, int flags);
/* TNNetSwiGLU (neural/neural.cl:1213-1263 flag 1): y[d] = x[d] * silu(x[half+d]). */
int cai_swiglu(const float* x, int half, int n_tokens, float* y, int flags);
/* ArgMaxRow (neural/neuralchatengine.pas:683-697): lowest index wins ties. */
int cai_argmax(const float* x, int n, int32_t* index_out, int flags);
/* cai_argmax for callers that cannot allocate device memory or wait (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc); it has no counterpart in the reference.  x_dev and index_out_dev are device pointers;
 * the two launches go to the library stream and the call returns without waiting.  The slice winners between the two
 * launches live in a fixed 8 KiB array inside the library (one copy per GPU, held until the process ends), which bounds
 * n at 4 194 304 (CAI_ERR_INVALID beyond).  Calls that overlap on one GPU share that array and race. */
int cai_argmax_noalloc(const float* x_dev, int n, int32_t* index_out_dev);
/* TNNetPointwiseSoftMax + TNNetTopKGate (neural/neuralpretrained.pas:15347-15365):
 * softmax over n experts, keep top-k, renormalise iff renorm.  Outputs are host arrays of k. */
int cai_router_topk(const float* logits, int n, int k, int renorm, int32_t* expert_out, float* gate_out, int flags);

/* =====================================================================================
 * KV cache + cached GQA decode attention (TNNetFusedSDPA).
 * Replaces BeginIncrementalDecode(MaxCtx, Int8KV) / ResetCache / TruncateCache / CacheLength /
 * Capture/RestoreCacheState (tests/TestNeuralFusedSDPA.pas:228-454) and the kernels
 * cai_sdpa_append_kv + cai_sdpa_decode (neural/neural.cl:2354-2499).
 * Cache layout is head-major: row (layer, kv_head g, position p) at ((layer*kv_heads+g)*max_ctx+p)*head_dim.
 * ===================================================================================== */
int cai_kv_create(int n_layers, int kv_heads, int head_dim, int max_ctx, int kv_dtype, cai_kv_t* out);
int cai_kv_destroy(cai_kv_t kv);
int cai_kv_reset(cai_kv_t kv);
int cai_kv_truncate(cai_kv_t kv, int n);          /* keeps the first n rows of every layer */
int cai_kv_len(cai_kv_t kv, int layer, int* len_out);   /* tokens appended so far = the next position */
/* StreamingLLM eviction (TNNetStreamingDecoder.EnableEviction / DisableEviction, neural/neuraldecode.pas:1257-1277,
 * 5722-5735): the first sink_tokens positions and the latest recent_window positions stay cached, the middle is
 * dropped, so a stream runs past max_ctx in constant memory.  Cached keys keep the rotation of their own position.
 * sink_tokens + recent_window <= max_ctx; 0, 0 turns it off.  Until the stream passes the cap, results are
 * bit-identical to the unbounded cache; the policy may only change while no sequence is past the smaller cap. */
int cai_kv_set_eviction(cai_kv_t kv, int sink_tokens, int recent_window);
int cai_kv_rows(cai_kv_t kv, int layer, int* rows_out);  /* rows held: min(len, cap) (SDPACacheLength, neural/neuraldecode.pas:1291-1294) */
int cai_kv_snapshot(cai_kv_t kv, cai_kv_snap_t* out);
int cai_kv_restore(cai_kv_t kv, cai_kv_snap_t snap);
int cai_kv_snap_destroy(cai_kv_snap_t snap);
/* Host copy of one layer's live rows and its inverse (CaptureCacheState / CaptureCacheStateInt8 and RestoreCacheState /
 * RestoreCacheStateInt8 as TNNetStreamingDecoder.Snapshot/Restore call them per layer, neural/neuraldecode.pas:5775-5790,
 * 5828-5840; also the hand-off of a host-built prefix to the device).  k and v hold [kv_heads][len][head_dim] elements
 * of the cache's type (float, IEEE half bits, or int8 codes); k_scales and v_scales hold [kv_heads][len] row scales and
 * are used only by a CAI_KV_I8 cache (null otherwise).  Import sets the layer's length to len. */
int cai_kv_export_layer(cai_kv_t kv, int layer, void* k, void* v, float* k_scales, float* v_scales);
int cai_kv_import_layer(cai_kv_t kv, int layer, int len, const void* k, const void* v, const float* k_scales, const float* v_scales);
/* One token of one layer: qkv = [Q (q_heads*hd) | K (kv_heads*hd) | V (kv_heads*hd)]; appends K,V at
 * slot CacheLength(layer), then out[h] = softmax(q_h.K/sqrt(hd)) V over the live range
 * (window > 0: last `window` rows; softcap > 0: Gemma-2 style cap).  out: [q_heads*hd]. */
int cai_attn_decode(cai_kv_t kv, int layer, const float* qkv, int q_heads, int window, float softcap,
                    float* out, int flags);

/* =====================================================================================
 * Step-resident decoder (TNNetStreamingDecoder over a Llama / Qwen2 / OLMoE graph).
 * Replaces Session.StepForward(InV, AbsPos) -> FNet.Compute (neural/neuraldecode.pas:5696-5712) for
 * the graph BuildLlamaFromTensorReaderWithConfig wires (neural/neuralpretrained.pas:16384-16882):
 * activations never leave the GPU inside a step (neural/tasklist.md:768-790 names the per-layer
 * host round trip as the bottleneck of the OpenCL path).
 * ===================================================================================== */
typedef struct cai_decoder_config {
  int32_t n_layers, d_model, n_q_heads, n_kv_heads, head_dim, ffn, vocab, max_ctx;
  float   eps, rope_theta;
  int32_t window;        /* sliding window, 0 = none */
  int32_t qk_norm_full;  /* OLMoE: RMSNorm over the full q and k widths before RoPE */
  int32_t n_experts;     /* 0 = dense SwiGLU FFN; else `ffn` is the per-expert width */
  int32_t top_k;
  int32_t norm_topk;
  int32_t kv_dtype;      /* CAI_KV_F32 / CAI_KV_F16 / CAI_KV_I8 */
  int32_t max_batch;     /* independent sequences, each with its own KV cache (1..8) */
} cai_decoder_config;

/* weight slots (layer = -1 for EMBED / HEAD; HEAD unset = tied to EMBED) */
#define CAI_W_EMBED  0
#define CAI_W_HEAD   1
#define CAI_W_Q      2
#define CAI_W_K      3
#define CAI_W_V      4
#define CAI_W_O      5
#define CAI_W_GATEUP 6  /* rows 0..I-1 up, I..2I-1 gate (neural/neuralpretrained.pas:240-243); MoE bank: expert e at rows e*2I */
#define CAI_W_DOWN   7  /* MoE bank: expert e at rows e*d_model */
#define CAI_W_ROUTER 8
/* vector slots */
#define CAI_V_ATTN_NORM  0
#define CAI_V_MLP_NORM   1
#define CAI_V_FINAL_NORM 2  /* layer = -1 */
#define CAI_V_Q_NORM     3
#define CAI_V_K_NORM     4

int cai_decoder_create(const cai_decoder_config* cfg, cai_decoder_t* out);
int cai_decoder_destroy(cai_decoder_t d);
/* The decoder borrows `w`; the caller destroys it after the decoder. q/k rows must be in the
 * interleaved-rotary order of MapTargetNeuron (neural/neuralpretrained.pas:14792-14812), which is the
 * stored order of llama.cpp GGUF files. */
int cai_decoder_set_weight(cai_decoder_t d, int layer, int slot, cai_qw_t w);
int cai_decoder_set_vector(cai_decoder_t d, int layer, int slot, const float* v_host, int n);
/* One token for each of sequences 0..n_b-1: tokens[b] at absolute position pos[b] (must equal that
 * sequence's cache length).  logits (host, [n_b][vocab]) and argmax (host, [n_b]) may be NULL. */
int cai_decoder_step(cai_decoder_t d, const int32_t* tokens, const int32_t* pos, int n_b,
                     float* logits, int32_t* argmax);
/* Width-n window step of ONE sequence (1 <= n <= 8): tokens[r] is fed at absolute position pos0 + r (pos0 = the cache
 * length), appended, and attends to everything before it; logits (host, [n][vocab]) and argmax (host, [n]) may be NULL, row r
 * is the output at position pos0 + r.  This is StepForward on a width-K twin (neural/neuraldecode.pas:1151-1183, 5696-5712),
 * the verify pass of speculative decoding (examples/SpeculativeDecoding/SpeculativeDecoding.lpr:646-663).  Afterwards the cache
 * holds pos0 + n rows; cai_decoder_truncate keeps the committed prefix (TruncateTo, neural/neuraldecode.pas:5714).  Sessions
 * with eviction take windows of one token only. */
int cai_decoder_step_window(cai_decoder_t d, int seq, const int32_t* tokens, int n, int pos0, float* logits, int32_t* argmax);
/* PromptLookupDraft (neural/neuraldecode.pas:7742-7765) on token ids: the tokens that followed the most recent earlier
 * occurrence of the context's last match_len tokens, at most num_draft of them (0: no earlier occurrence).  Host only. */
int cai_prompt_lookup_draft(const int32_t* context, int n_ctx, int match_len, int num_draft, int32_t* draft_out, int* n_draft_out);
/* DecodePromptLookup (neural/neuraldecode.pas:7767-7866) on the cached session: greedy continuation of sequence 0 whose passes
 * verify a prompt-lookup draft of up to min(num_draft, 7) tokens in one window step.  context[0 .. n_ctx-2] must be in the
 * cache; context[n_ctx-1] is fed first.  Writes n_tokens ids - the ones cai_decoder_generate would write - and the number of
 * passes taken (may be NULL); the cache ends n_ctx - 1 + n_tokens rows long. */
int cai_decoder_generate_lookup(cai_decoder_t d, const int32_t* context, int n_ctx, int match_len, int num_draft,
                                int n_tokens, int32_t* tokens_out, int32_t* passes_out);
/* HiddenState of the session (neural/neuraldecode.pas:1314-1321, 5850-5857): the input of the vocabulary projection, i.e. the
 * final RMSNorm of the residual stream, d_model floats (host), for row `row` (0..7) of the last step or window; row 0 after
 * cai_decoder_prefill and cai_decoder_generate (the last token fed).  What contrastive search and embedding consumers read. */
int cai_decoder_hidden_state(cai_decoder_t d, int row, float* hidden_out);
/* Greedy continuation of sequence 0 with no host round trip between tokens: feeds `first_token` at
 * position `pos`, then each argmax as the next token; writes n_tokens ids (the greedy fast path of
 * neural/neuralchatengine.pas:1485-1561 with ArgMaxRow on the device). */
int cai_decoder_generate(cai_decoder_t d, int32_t first_token, int pos, int n_tokens, int32_t* tokens_out);
/* Measurement aid (no counterpart in the reference): average microseconds per step spent in each kernel class of the batch-1
 * decode step of sequence 0 at its current position, taken as a difference: `reps` whole steps, and `reps` steps without class
 * k's launches, each captured and replayed as one graph between two HIP events on the library stream; a class costs what the
 * step gains without it (the kernel in its place in the chain, dependent-launch gap included; the classes add up to the step).
 * Classes: 0 embedding, 1 q|k|v, 2 attention (rotary + append + cached decode), 3 o + residual,
 * 4 RMSNorm + gate|up + SwiGLU (expert half of a mixture model: router .. mixture, with 5), 5 down + residual, 6 final norm +
 * vocabulary projection, 7 arg-max.  The session is not advanced (the K,V row of the current position is rewritten). */
int cai_decoder_profile(cai_decoder_t d, int32_t token, int reps, float* us_per_step_out, int n_classes);
/* Measurement aid (no counterpart in the reference): device-side timeline of ONE batch-1 decode step of sequence 0 at its current
 * position.  The step is captured with timeline records armed and replayed as a graph three times; the stamps of the last
 * replay come back.  Instrumented launches (the integer-dot and block matrix-vector kernels, the per-head attention kernel)
 * store eight wall-clock stamps per work-group (thread 0): 0 entry, 7 exit (after the result stores were issued), 4 inputs
 * staged (activation in registers / query rotated), 5 main loop done; matrix-vector kernels also 1 first requests issued,
 * 2 activation values arrived, 3 block-float form complete in LDS; attention also 1 position known, 6 arrival counted.  A stamp a
 * work-group never reached stays zero.  launches_out[3 i ..] = class of launch i (as in cai_decoder_profile), its
 * work-groups, index of its first stamp; stamps_out[first + 8 wg + k].  ticks_per_us_out: wall-clock ticks per microsecond.
 * The session is not advanced. */
int cai_decoder_timeline(cai_decoder_t d, int32_t token, uint64_t* stamps_out, int64_t stamps_cap, int32_t* launches_out,
                         int launches_cap, int* n_launches_out, int64_t* n_stamps_out, float* ticks_per_us_out);
/* Multi-token prompt ingestion for sequence `seq` on the matrix cores: equals n sequential steps
 * within tolerance.  last_logits (host, [vocab]) and argmax may be NULL. */
int cai_decoder_prefill(cai_decoder_t d, int seq, const int32_t* tokens, int n, int pos0,
                        float* last_logits, int32_t* argmax);
/* Session management (neural/neuraldecode.pas:5714-5843): always safe after a failed step. */
/* ---- distribution pipeline ahead of the samplers, on the device ----
 * The non-greedy branch of TChatEngine.GenerateFromIds (neural/neuralchatengine.pas:1374-1396, 1495-1501): RowSoftMax ->
 * TNNetPenaltyProcessor (ApplyToProbabilities, neural/neuralvolume.pas:5335-5376) -> TNNetTemperatureProcessor
 * (neural/neuraldecode.pas:4710-4754) -> the candidate prefix the samplers draw from (SelectTopCandidates +
 * SortTokenArray, neural/neuralvolume.pas:5171-5196): the m <= 1024 most probable tokens, descending, equal
 * probabilities by token id.  hist_ids / hist_counts: the DISTINCT tokens of the context and how often each occurred
 * (TNNetTokenHistoryPenalty's FSeen / FCounts); repetition 1, frequency 0, presence 0, temperature 1 are no-ops.
 * The draw (uniform over the window for TopK / TopP, weighted for WeightedTopK / MinP) stays with the host and its
 * random generator.  *count_out = min(m, n).  cai_decoder_candidates reads logits row `row` (0..7) of the session's last
 * step (row = sequence) or window (row = position in the window) in place, with no read-back of the row (after a prompt pass
 * and after cai_decoder_generate: row 0); cai_sample_candidates takes any row (CAI_X_DEVICE: a device pointer). */
int cai_sample_candidates(const float* logits, int n, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                          float repetition, float frequency, float presence, float temperature, int m,
                          int32_t* tokens_out, float* probs_out, int* count_out, int flags);
int cai_decoder_candidates(cai_decoder_t d, int row, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                           float repetition, float frequency, float presence, float temperature, int m,
                           int32_t* tokens_out, float* probs_out, int* count_out);
int cai_decoder_reset(cai_decoder_t d, int seq);
int cai_decoder_truncate(cai_decoder_t d, int seq, int n);
int cai_decoder_len(cai_decoder_t d, int seq, int* len_out);   /* tokens streamed so far = the next position */
/* Eviction for every layer of every sequence of the session (see cai_kv_set_eviction); with it on, positions may run
 * past max_ctx.  cai_decoder_cache_rows is SDPACacheLength(Index) (neural/neuraldecode.pas:1291-1294). */
int cai_decoder_set_eviction(cai_decoder_t d, int sink_tokens, int recent_window);
int cai_decoder_cache_rows(cai_decoder_t d, int seq, int layer, int* rows_out);
/* EnableInt8KVCache / DisableInt8KVCache (neural/neuraldecode.pas:1277-1290): switches the cache element type; like the
 * reference only on an empty session (CAI_ERR_STATE once a token has been streamed). */
int cai_decoder_set_kv_dtype(cai_decoder_t d, int kv_dtype);
/* Long-context rules of TNNetRotaryEmbedding as the importers set them from "rope_scaling" (neural/neuralpretrained.pas:633-668,
 * 13365, 13425): CAI_ROPE_LINEAR = Position Interpolation (theta_k / factor), CAI_ROPE_LLAMA3 = the Llama-3.1 rule
 * (original_ctx, low_freq_factor, high_freq_factor; no output scale).  Both only change the frequency table, which is rebuilt
 * in double on the host.  Only on an empty session (CAI_ERR_STATE otherwise: cached keys carry the old rotation). */
#define CAI_ROPE_NONE   0
#define CAI_ROPE_LINEAR 1
#define CAI_ROPE_LLAMA3 2
#define CAI_ROPE_NTK    3  /* "dynamic" / "ntk": base * factor^(d/(d-2)) */
#define CAI_ROPE_YARN   4  /* low_freq_factor = beta_slow (YarnAlpha), high_freq_factor = beta_fast (YarnBeta); sets the output scale 0.1 ln(factor) + 1 */
int cai_decoder_set_rope_scaling(cai_decoder_t d, int mode, float factor, int original_ctx, float low_freq_factor, float high_freq_factor);
/* Per-frequency divisors: theta_k = base^(-2k/head_dim) / factors[k], n = head_dim / 2 (the "rope_freqs.weight" tensor llama.cpp
 * writes for Llama-3.1 exports; the LongFactors table of the reference's record, neural/neuralpretrained.pas:652-655). */
int cai_decoder_set_rope_freq_factors(cai_decoder_t d, const float* factors, int n);
/* The factor the rotary layer puts on its output (YaRN temperature, an explicit attention_factor, LongRoPE's LongAttnFactor:
 * neural/neuralpretrained.pas:656-667).  The layer sits on q and k, so the session multiplies the attention scores by
 * scale^2 instead and caches K unscaled.  cai_decoder_set_rope_scaling sets it (YaRN: 0.1 ln(factor) + 1, else 1); call this
 * afterwards to override.  Empty session only. */
int cai_decoder_set_rope_out_scale(cai_decoder_t d, float scale);
int cai_decoder_snapshot(cai_decoder_t d, int seq, cai_kv_snap_t* out);
int cai_decoder_restore(cai_decoder_t d, int seq, cai_kv_snap_t snap);
/* Sequence dst_seq becomes a copy of src_seq (rows and length), device to device on the library's stream: the cache fork of a
 * beam search, whose survivors each continue from their parent's cache (DecodeBeamSearchCachedAll, neural/neuraldecode.pas:1436-1453,
 * keeps one snapshot per hypothesis instead).  The beams of a step are then ONE cai_decoder_step over the sequences. */
int cai_decoder_fork(cai_decoder_t d, int src_seq, int dst_seq);
/* Bytes of weights, biases and gains one decoded token streams (for roofline accounting). */
/* the configuration the decoder was created with (a loader fills it from the file) */
int cai_decoder_get_config(cai_decoder_t d, cai_decoder_config* out);
int cai_decoder_weight_bytes(cai_decoder_t d, int64_t* algorithmic_bytes_out);

/* ---------------------------------------------------------------------------------------------
 * GGUF container (replaces TNNetGGUFReader, neural/neuralgguf.pas:1072-1220 ParseFile, 1525-1672 tensor reads)
 * and the llama / qwen2 importer (BuildLlamaFromGGUFEx and the qwen2 branch, neural/neuralpretrained.pas:17484-17876).
 * The file is mapped read-only.  Shapes are row-major (ggml's contiguous axis last): an HF [out, in] matrix reads
 * [out, in].  Tokenizer metadata stays with the host application.
 * ------------------------------------------------------------------------------------------- */
typedef struct cai_gguf_s* cai_gguf_t;
int cai_gguf_open(const char* path, cai_gguf_t* out);
int cai_gguf_close(cai_gguf_t g);
int cai_gguf_info(cai_gguf_t g, int* version, int* alignment, int64_t* n_tensors, int64_t* n_meta, int64_t* data_start);
int cai_gguf_meta_int(cai_gguf_t g, const char* key, int64_t* out);      /* GetMetaInt: any integer or bool value */
int cai_gguf_meta_float(cai_gguf_t g, const char* key, double* out);     /* GetMetaFloat */
int cai_gguf_meta_str(cai_gguf_t g, const char* key, char* buf, int n);  /* GetMetaString */
int cai_gguf_meta_array_count(cai_gguf_t g, const char* key, int64_t* out);
int cai_gguf_meta_array_str(cai_gguf_t g, const char* key, int64_t index, char* buf, int n);  /* GetMetaArrayString */
int cai_gguf_find_tensor(cai_gguf_t g, const char* name, int64_t* index);
int cai_gguf_tensor_info(cai_gguf_t g, int64_t index, char* name_buf, int name_n, int* ggml_type, int* n_dims,
                         int64_t* shape8, int64_t* data_offset, int64_t* nbytes);
/* pointer into the mapping, valid until cai_gguf_close (the raw-bytes read of neural/neuralsafetensors.pas:1024) */
int cai_gguf_tensor_data(cai_gguf_t g, int64_t index, const void** ptr);
/* resident weight from a 2-D tensor in stored order and stored type (F32, F16, Q4_0, Q8_0, Q4_K, Q6_K); bias_name may be
 * NULL or name a tensor that is absent */
int cai_gguf_load_qw(cai_gguf_t g, const char* name, const char* bias_name, cai_qw_t* out);
/* Whole decoder from a llama or qwen2 file; the decoder owns the weights it loads.  max_ctx <= 0 takes
 * <arch>.context_length.  Blocks go up in stored order: llama.cpp's q/k row order is the interleaved-rotary order
 * the decode kernels rotate (neural/neuralgguf.pas:428-438 composed with neural/neuralpretrained.pas:14792-14812
 * is the identity). */
int cai_decoder_load_gguf(const char* path, int max_ctx, int max_batch, int kv_dtype, cai_decoder_t* out);

#ifdef __cplusplus
}
#endif
#endif
