{
  caihip.pas - Free Pascal binding of libcaihip.so (include/caihip.h), the MI355X (gfx950)
  quantized decode path for CAI Neural API.

  Declarative unit: cdecl externals + constants, no logic.  It mirrors the role of the OpenCL
  bindings the reference uses for its offload object (neural/neuralopencl.pas:245-388).
  Not compiled in this repository's CI (no fpc in the build image); the C header is authoritative.
  Pascal owns host volumes (pass @Volume.FData[0] and lengths); the library owns device memory.
}
unit caihip;

{$mode objfpc}{$H+}

interface

const
  CAIHIP_LIB = 'caihip';

  CAI_OK = 0; CAI_ERR_INVALID = -1; CAI_ERR_HIP = -2; CAI_ERR_NOMEM = -3;
  CAI_ERR_UNSUPPORTED = -4; CAI_ERR_STATE = -5;

  // ggml tensor type ids (neural/neuralgguf.pas:86-98) + per-row int8
  CAI_F32 = 0; CAI_F16 = 1; CAI_Q4_0 = 2; CAI_Q8_0 = 8; CAI_Q4_K = 12; CAI_Q6_K = 14; CAI_I8ROW = 100;
  CAI_Q4_1 = 3; CAI_Q5_0 = 6; CAI_Q5_1 = 7; CAI_Q2_K = 10; CAI_Q3_K = 11; CAI_Q5_K = 13;
  CAI_ROPE_NONE = 0; CAI_ROPE_LINEAR = 1; CAI_ROPE_LLAMA3 = 2; CAI_ROPE_NTK = 3; CAI_ROPE_YARN = 4;
  // fused activation opcodes = csAct* of the OpenCL kernels (neural/neural.cl:114-146)
  CAI_ACT_NONE = 0; CAI_ACT_RELU = 1; CAI_ACT_SIGMOID = 2; CAI_ACT_TANH = 3;
  CAI_X_DEVICE = 1; CAI_Y_DEVICE = 2; CAI_MATRIX_CORES = 4;
  CAI_KV_F32 = 0; CAI_KV_F16 = 1; CAI_KV_I8 = 2;
  CAI_W_EMBED = 0; CAI_W_HEAD = 1; CAI_W_Q = 2; CAI_W_K = 3; CAI_W_V = 4; CAI_W_O = 5;
  CAI_W_GATEUP = 6; CAI_W_DOWN = 7; CAI_W_ROUTER = 8;
  CAI_V_ATTN_NORM = 0; CAI_V_MLP_NORM = 1; CAI_V_FINAL_NORM = 2; CAI_V_Q_NORM = 3; CAI_V_K_NORM = 4;

type
  TCaiQW = Pointer; TCaiKV = Pointer; TCaiKVSnap = Pointer; TCaiDecoder = Pointer; TCaiGGUF = Pointer;
  PCaiQW = ^TCaiQW; PCaiKV = ^TCaiKV; PCaiKVSnap = ^TCaiKVSnap; PCaiDecoder = ^TCaiDecoder; PCaiGGUF = ^TCaiGGUF;

  TCaiDecoderConfig = packed record
    n_layers, d_model, n_q_heads, n_kv_heads, head_dim, ffn, vocab, max_ctx: LongInt;
    eps, rope_theta: Single;
    window, qk_norm_full, n_experts, top_k, norm_topk, kv_dtype, max_batch: LongInt;
  end;
  PCaiDecoderConfig = ^TCaiDecoderConfig;

function cai_init(device_ordinal: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_shutdown(): LongInt; cdecl; external CAIHIP_LIB;
function cai_last_error(buf: PAnsiChar; buf_len: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_device_name(buf: PAnsiChar; buf_len: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_sync(): LongInt; cdecl; external CAIHIP_LIB;
function cai_get_stream(stream_out: PPointer): LongInt; cdecl; external CAIHIP_LIB;
function cai_timer_start(): LongInt; cdecl; external CAIHIP_LIB;
function cai_timer_stop(ms_out: PSingle): LongInt; cdecl; external CAIHIP_LIB;
function cai_dev_alloc(bytes: Int64; ptr_out: PPointer): LongInt; cdecl; external CAIHIP_LIB;
function cai_dev_free(ptr: Pointer): LongInt; cdecl; external CAIHIP_LIB;
function cai_dev_upload(dst_dev, src_host: Pointer; bytes: Int64): LongInt; cdecl; external CAIHIP_LIB;
function cai_dev_download(dst_host, src_dev: Pointer; bytes: Int64): LongInt; cdecl; external CAIHIP_LIB;
function cai_dev_copy(dst_dev, src_dev: Pointer; bytes: Int64): LongInt; cdecl; external CAIHIP_LIB;

function cai_qw_create(qtype: LongInt; rows, cols: Int64; blocks: Pointer; bias: PSingle; out_w: PCaiQW): LongInt; cdecl; external CAIHIP_LIB;
function cai_qw_create_int8row(rows, cols: Int64; codes: PShortInt; scales, bias: PSingle; out_w: PCaiQW): LongInt; cdecl; external CAIHIP_LIB;
function cai_qw_destroy(w: TCaiQW): LongInt; cdecl; external CAIHIP_LIB;
function cai_qw_info(w: TCaiQW; qtype: PLongInt; rows, cols, device_bytes: PInt64): LongInt; cdecl; external CAIHIP_LIB;
function cai_qw_dequant_rows(w: TCaiQW; row0, n_rows: Int64; out_f: PSingle; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_qgemv(w: TCaiQW; x: PSingle; n_b: LongInt; y: PSingle; act, flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_ffn_gateup(gateup: TCaiQW; x, gain: PSingle; eps: Single; n_b: LongInt; y: PSingle; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_qgemm(w: TCaiQW; x: PSingle; n_tokens: LongInt; y: PSingle; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;

function cai_rmsnorm(x, gain_host: PSingle; n, n_tokens: LongInt; eps: Single; y: PSingle; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_rope(x: PSingle; n_heads, head_dim, pos: LongInt; theta_base: Single; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_swiglu(x: PSingle; half, n_tokens: LongInt; y: PSingle; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_argmax(x: PSingle; n: LongInt; index_out: PLongInt; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_argmax_noalloc(x_dev: PSingle; n: LongInt; index_out_dev: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_router_topk(logits: PSingle; n, k, renorm: LongInt; expert_out: PLongInt; gate_out: PSingle; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;

function cai_kv_create(n_layers, kv_heads, head_dim, max_ctx, kv_dtype: LongInt; out_kv: PCaiKV): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_destroy(kv: TCaiKV): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_reset(kv: TCaiKV): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_truncate(kv: TCaiKV; n: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_len(kv: TCaiKV; layer: LongInt; len_out: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_snapshot(kv: TCaiKV; out_snap: PCaiKVSnap): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_restore(kv: TCaiKV; snap: TCaiKVSnap): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_snap_destroy(snap: TCaiKVSnap): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_set_eviction(kv: TCaiKV; sink_tokens, recent_window: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_rows(kv: TCaiKV; layer: LongInt; rows_out: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_export_layer(kv: TCaiKV; layer: LongInt; k, v: Pointer; k_scales, v_scales: PSingle): LongInt; cdecl; external CAIHIP_LIB;
function cai_kv_import_layer(kv: TCaiKV; layer, len: LongInt; k, v: Pointer; k_scales, v_scales: PSingle): LongInt; cdecl; external CAIHIP_LIB;
function cai_attn_decode(kv: TCaiKV; layer: LongInt; qkv: PSingle; q_heads, window: LongInt; softcap: Single; out_f: PSingle; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;

function cai_decoder_create(cfg: PCaiDecoderConfig; out_d: PCaiDecoder): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_destroy(d: TCaiDecoder): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_set_weight(d: TCaiDecoder; layer, slot: LongInt; w: TCaiQW): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_set_vector(d: TCaiDecoder; layer, slot: LongInt; v_host: PSingle; n: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_step(d: TCaiDecoder; tokens, pos: PLongInt; n_b: LongInt; logits: PSingle; argmax: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_hidden_state(d: TCaiDecoder; row: LongInt; hidden_out: PSingle): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_step_window(d: TCaiDecoder; seq: LongInt; tokens: PLongInt; n, pos0: LongInt; logits: PSingle; argmax: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_prompt_lookup_draft(context: PLongInt; n_ctx, match_len, num_draft: LongInt; draft_out: PLongInt; n_draft_out: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_generate_lookup(d: TCaiDecoder; context: PLongInt; n_ctx, match_len, num_draft, n_tokens: LongInt; tokens_out: PLongInt; passes_out: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_generate(d: TCaiDecoder; first_token, pos, n_tokens: LongInt; tokens_out: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_profile(d: TCaiDecoder; token, reps: LongInt; us_per_step_out: PSingle; n_classes: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_timeline(d: TCaiDecoder; token: LongInt; stamps_out: PQWord; stamps_cap: Int64; launches_out: PLongInt; launches_cap: LongInt; n_launches_out: PLongInt; n_stamps_out: PInt64; ticks_per_us_out: PSingle): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_prefill(d: TCaiDecoder; seq: LongInt; tokens: PLongInt; n, pos0: LongInt; last_logits: PSingle; argmax: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_reset(d: TCaiDecoder; seq: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_truncate(d: TCaiDecoder; seq, n: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_sample_candidates(logits: PSingle; n: LongInt; hist_ids, hist_counts: PLongInt; n_hist: LongInt;
  repetition, frequency, presence, temperature: Single; m: LongInt; tokens_out: PLongInt; probs_out: PSingle;
  count_out: PLongInt; flags: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_candidates(d: TCaiDecoder; row: LongInt; hist_ids, hist_counts: PLongInt; n_hist: LongInt;
  repetition, frequency, presence, temperature: Single; m: LongInt; tokens_out: PLongInt; probs_out: PSingle;
  count_out: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_len(d: TCaiDecoder; seq: LongInt; len_out: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_set_eviction(d: TCaiDecoder; sink_tokens, recent_window: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_set_kv_dtype(d: TCaiDecoder; kv_dtype: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_set_rope_scaling(d: TCaiDecoder; mode: LongInt; factor: Single; original_ctx: LongInt; low_freq_factor, high_freq_factor: Single): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_set_rope_freq_factors(d: TCaiDecoder; factors: PSingle; n: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_set_rope_out_scale(d: TCaiDecoder; scale: Single): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_cache_rows(d: TCaiDecoder; seq, layer: LongInt; rows_out: PLongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_snapshot(d: TCaiDecoder; seq: LongInt; out_snap: PCaiKVSnap): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_restore(d: TCaiDecoder; seq: LongInt; snap: TCaiKVSnap): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_fork(d: TCaiDecoder; src_seq, dst_seq: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_weight_bytes(d: TCaiDecoder; algorithmic_bytes_out: PInt64): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_get_config(d: TCaiDecoder; out_cfg: Pointer): LongInt; cdecl; external CAIHIP_LIB;
function cai_decoder_load_gguf(path: PChar; max_ctx, max_batch, kv_dtype: LongInt; out_decoder: PCaiDecoder): LongInt; cdecl; external CAIHIP_LIB;

// GGUF container (TNNetGGUFReader, neural/neuralgguf.pas:1072-1220)
function cai_gguf_open(path: PChar; out_gguf: PCaiGGUF): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_close(g: TCaiGGUF): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_info(g: TCaiGGUF; version, alignment: PLongInt; n_tensors, n_meta, data_start: PInt64): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_meta_int(g: TCaiGGUF; key: PChar; out_value: PInt64): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_meta_float(g: TCaiGGUF; key: PChar; out_value: PDouble): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_meta_str(g: TCaiGGUF; key: PChar; buf: PChar; n: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_meta_array_count(g: TCaiGGUF; key: PChar; out_count: PInt64): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_meta_array_str(g: TCaiGGUF; key: PChar; index: Int64; buf: PChar; n: LongInt): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_find_tensor(g: TCaiGGUF; name: PChar; index: PInt64): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_tensor_info(g: TCaiGGUF; index: Int64; name_buf: PChar; name_n: LongInt; ggml_type, n_dims: PLongInt; shape8, data_offset, nbytes: PInt64): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_tensor_data(g: TCaiGGUF; index: Int64; ptr: PPointer): LongInt; cdecl; external CAIHIP_LIB;
function cai_gguf_load_qw(g: TCaiGGUF; name, bias_name: PChar; out_qw: PCaiQW): LongInt; cdecl; external CAIHIP_LIB;

implementation

end.
