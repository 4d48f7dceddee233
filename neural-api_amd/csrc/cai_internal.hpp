// Internal declarations shared by the caihip translation units (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <string>
#include <vector>

#include "../../include/caihip.h"

namespace cai {

struct Context {
  bool        ready = false;
  int         device = 0;
  hipStream_t stream = nullptr;
  hipEvent_t  ev0 = nullptr, ev1 = nullptr;
  int         n_cu = 256;
  char        name[128] = {0};
  // scratch used by calls that take host pointers (grown on demand)
  void*  stage_in = nullptr;  size_t stage_in_cap = 0;
  void*  stage_out = nullptr; size_t stage_out_cap = 0;
  void*  stage_sample = nullptr; size_t stage_sample_cap = 0;   // a host logits row on its way to cai_sample_candidates
  int32_t* d_small = nullptr;            // 1024 ints of device scratch for small arguments/results
  int32_t* h_small = nullptr;            // 1024 ints of pinned host memory paired with d_small
  // Step timeline (measurement aid, cai_decoder_timeline): while armed, every instrumented launch gets a record of eight
  // wall-clock stamps per work-group (0 entry .. 7 exit, the ones between are the kernel's own) and a descriptor (class,
  // work-groups, offset)
  struct Timeline {
    bool armed = false; int cls = 0;
    unsigned long long* buf = nullptr; size_t cap = 0, used = 0;   // stamps (device)
    std::vector<int32_t> launches;                                  // [n][3]: class, work-groups, first stamp
  } tl;
};
// record of the launch being enqueued (null unless a timeline is armed): TL_STAMPS stamps per work-group.  The stamps exist
// only in a build with -DCAI_TIMELINE (make timeline -> libcaihip_timeline.so): even a never-taken stamp costs the streaming
// kernels 3 % (the branch around it makes the compiler wait for every outstanding request where the paths join).
constexpr int TL_STAMPS = 8;
unsigned long long* timeline_next(int n_wg);
#ifdef CAI_TIMELINE
__device__ __forceinline__ void timeline_stamp(unsigned long long* t, int k)
{
  if (t && threadIdx.x == 0) t[(size_t)(blockIdx.x + gridDim.x * blockIdx.y) * TL_STAMPS + k] = wall_clock64();
}
// entry stamp: taken into a register before anything is fetched (the record's address comes from the argument block, which
// is a memory round trip away at that point) and stored with timeline_put once the first requests are out
__device__ __forceinline__ unsigned long long timeline_now() { return wall_clock64(); }
__device__ __forceinline__ void timeline_put(unsigned long long* t, int k, unsigned long long v)
{
  if (t && threadIdx.x == 0) t[(size_t)(blockIdx.x + gridDim.x * blockIdx.y) * TL_STAMPS + k] = v;
}
// the same once `dep` has arrived (a stamp the compiler may not move in front of the wait for a loaded value)
__device__ __forceinline__ void timeline_stamp_after(unsigned long long* t, int k, float dep)
{
  if (t) { asm volatile("" :: "v"(dep)); timeline_stamp(t, k); }
}
#else
__device__ __forceinline__ void timeline_stamp(unsigned long long*, int) {}
__device__ __forceinline__ unsigned long long timeline_now() { return 0; }
__device__ __forceinline__ void timeline_put(unsigned long long*, int, unsigned long long) {}
__device__ __forceinline__ void timeline_stamp_after(unsigned long long*, int, float) {}
#endif

Context& ctx();
struct ApiLock { ApiLock(); ~ApiLock(); ApiLock(const ApiLock&) = delete; ApiLock& operator=(const ApiLock&) = delete; };
int  set_error(int code, const char* fmt, ...);
int  hip_fail(hipError_t e, const char* what, const char* file, int line);
int  ensure_stage(void** p, size_t* cap, size_t need);

#define CAI_HIP(call)                                                        \
  do {                                                                       \
    hipError_t e__ = (call);                                                 \
    if (e__ != hipSuccess) return cai::hip_fail(e__, #call, __FILE__, __LINE__); \
  } while (0)

#define CAI_REQUIRE(cond, ...)                                               \
  do {                                                                       \
    if (!(cond)) return cai::set_error(CAI_ERR_INVALID, __VA_ARGS__);        \
  } while (0)

// first statement of every exported function: calls from several host threads are serialised
#define CAI_ENTER() cai::ApiLock api_lock__

#define CAI_READY()                                                          \
  do {                                                                       \
    if (!cai::ctx().ready) return cai::set_error(CAI_ERR_STATE, "cai_init has not been called"); \
  } while (0)

// x = hi + lo for a pair of f16 operands (22 significant bits).  hi is rounded to 11 significant bits on the float's own
// bit pattern (nearest even), so its conversion to f16 is exact whichever conversion instruction the compiler picks for
// the scalar and for the packed use of the value (the two were seen to disagree in rare cases); lo = x - hi is exact in
// fp32.  NaN and Inf stay what they are (lo of an Inf is NaN: still poison).
__device__ __forceinline__ void split_f16(float x, _Float16& hi, _Float16& lo)
{
  const uint32_t b = __builtin_bit_cast(uint32_t, x);
  const float h = __builtin_bit_cast(float, (b + 0xFFFu + ((b >> 13) & 1u)) & 0xFFFFE000u);
  hi = (_Float16)h; lo = (_Float16)(x - h);
}

// Walks x[i0], x[i0 + step], ... (< n, n >= 1) and hands every value to f(value, index) in index order.  Eight requests go out
// before the first value is used: a loop that uses each value as it arrives pays one cache round trip per element, which is
// what a 256-thread work-group reducing a few thousand activations otherwise spends most of its time on.  The second form
// walks two arrays side by side (g may be null: its values are then 1).
template <typename F>
__device__ __forceinline__ void for_strided8(const float* x, int i0, int n, int step, F f)
{
  for (int i = i0; i < n; i += 8 * step) {
    float t[8];
#pragma unroll
    for (int u = 0; u < 8; u++) t[u] = x[min(i + u * step, n - 1)];
#pragma unroll
    for (int u = 0; u < 8; u++) if (i + u * step < n) f(t[u], i + u * step);
  }
}
template <typename F>
__device__ __forceinline__ void for_strided8(const float* x, const float* g, int i0, int n, int step, F f)
{
  for (int i = i0; i < n; i += 8 * step) {
    float t[8], tg[8];
#pragma unroll
    for (int u = 0; u < 8; u++) { const int j = min(i + u * step, n - 1); t[u] = x[j]; tg[u] = g ? g[j] : 1.0f; }
#pragma unroll
    for (int u = 0; u < 8; u++) if (i + u * step < n) f(t[u], tg[u], i + u * step);
  }
}

// ---------------------------------------------------------------------------------------------
// Resident weight matrix.  Device layouts (the on-disk block format stays the contract; these are
// the library's own):
//   Q4_K : the 144-byte super-blocks as stored (16-byte aligned rows).
//   Q8_0 : two planes - qs[rows][cols] int8 (32 B per block, 16-byte aligned) and d[rows][cols/32] half.
//   Q4_0 : two planes - qs[rows][cols/2] bytes (16 B per block) and d[rows][cols/32] half.
//   F32/F16 : as stored.   I8ROW : codes[rows][cols] + scales[rows].
// ---------------------------------------------------------------------------------------------
}  // namespace cai

struct cai_qw_s {
  int      qtype = 0;
  int64_t  rows = 0, cols = 0;
  uint8_t* data = nullptr;     // quants plane or the raw blocks
  uint8_t* aux = nullptr;      // half scales plane (Q8_0/Q4_0), float row scales (I8ROW), or for Q6_K the int8 scales plane (16 per block) followed by the plane of d
  float*   bias = nullptr;
  int64_t  data_bytes = 0, aux_bytes = 0;
  int64_t  algo_bytes = 0;     // bytes of the GGUF form (+bias): what one GEMV must stream
};

// The block types that stay resident as the stored block stream (no repacking at upload)
__host__ __device__ constexpr bool raw_block_type(int qt)
{
  return qt == CAI_Q4_1 || qt == CAI_Q5_0 || qt == CAI_Q5_1 || qt == CAI_Q2_K || qt == CAI_Q3_K || qt == CAI_Q5_K;
}
__host__ __device__ constexpr int raw_block_bytes(int qt)
{
  return qt == CAI_Q4_1 ? 20 : qt == CAI_Q5_0 ? 22 : qt == CAI_Q5_1 ? 24 : qt == CAI_Q2_K ? 84 : qt == CAI_Q3_K ? 110 : qt == CAI_Q5_K ? 176 : 0;
}
__host__ __device__ constexpr int raw_block_elems(int qt) { return (qt == CAI_Q2_K || qt == CAI_Q3_K || qt == CAI_Q5_K) ? 256 : 32; }

// Q6_K: start of the d plane (behind 16 scale bytes per block); null for the other types
inline const uint8_t* qw_aux2(const cai_qw_s* w) { return w->qtype == CAI_Q6_K ? w->aux + w->rows * (w->cols >> 8) * 16 : nullptr; }

struct cai_kv_s {
  int n_seq = 1, n_layers = 0, kv_heads = 0, head_dim = 0, max_ctx = 0, dtype = 0;
  float score_mul = 1.0f;                 // on top of 1 / sqrt(head_dim): the square of the rotary layer's output scale
  void* k = nullptr; void* v = nullptr;   // [seq][layer][kv_head][max_ctx][head_dim]
  float* ks = nullptr; float* vs = nullptr;   // CAI_KV_I8 only: one scale per cached row, [seq][layer][kv_head][max_ctx]
  std::vector<int> len;                   // [seq][layer] stream position = tokens appended so far (host mirror)
  int evict_sinks = 0, evict_cap = 0;     // cap > 0: sink + recent-window eviction, at most cap rows are cached
  int live(int n) const { return evict_cap > 0 && n > evict_cap ? evict_cap : n; }   // cached rows after n tokens
  int split_len = 64, n_splits = 1;       // slice geometry of the decode kernels for a cache filled up to max_ctx
  int n_splits_alloc = 1;                 // most slices any length bucket uses (sizes the per-slice scratch)
  int geo_rows = 0;                       // rows the launches being enqueued must cover (0: max_ctx); see kv_geometry
  float* part = nullptr;                  // [seq][q_head][split][head_dim+2] split-K partials
  int part_q_heads = 0;
  int32_t* d_len = nullptr;               // [seq] device scratch: rows live BEFORE the token being decoded
  unsigned* merge_cnt = nullptr;          // [seq][part_q_heads] arrival counters of the in-kernel merge of the split partials (wrap to 0 by themselves)
  void* pq_hi = nullptr; void* pq_lo = nullptr; size_t pq_cap = 0;   // prompt ingestion: rotated q of a chunk as two f16 planes
  float* pq_part = nullptr; size_t pq_part_cap = 0;                     // prompt ingestion: partial results of a token tile's K splits
  size_t elem() const { return dtype == CAI_KV_F16 ? 2 : dtype == CAI_KV_I8 ? 1 : 4; }
  int64_t layer_rows() const { return (int64_t)kv_heads * max_ctx; }
  int64_t seq_rows() const { return layer_rows() * n_layers; }
  int64_t layer_elems() const { return (int64_t)kv_heads * max_ctx * head_dim; }
  int64_t seq_elems() const { return layer_elems() * n_layers; }
  int& len_at(int seq, int layer) { return len[(size_t)seq * n_layers + layer]; }
};

struct cai_kv_snap_s {
  int n_layers = 0, kv_heads = 0, head_dim = 0, dtype = 0, rows = 0;
  int evict_sinks = 0, evict_cap = 0;     // the eviction policy the rows were laid out under
  std::vector<int> len;                   // per layer
  void* k = nullptr; void* v = nullptr;   // [layer][kv_head][rows][head_dim]
  float* ks = nullptr; float* vs = nullptr;   // [layer][kv_head][rows] row scales of an int8 cache
};

namespace cai {

// ---- launchers (all enqueue on ctx().stream; pointers are device pointers) ----
int launch_gemv(const cai_qw_s* w, int64_t row0, int64_t n_rows, const float* x, int n_b, float* y,
                int64_t y_stride, int act, const float* residual);
// Up to three matrices of one type and width sharing the staged activation (q|k|v in one launch); or, with
// slot_expert set, n_slots row windows of one expert bank (window e = rows [e*expert_rows, +rows[0]) ), slot j
// reading x + j*x_slot_stride and writing y + j*y_slot_stride.
struct MultiGemv {
  const cai_qw_s* w[3]; int64_t row0[3]; int64_t rows[3]; int y_off[3]; int n;
  const int32_t* slot_expert; int n_slots; int64_t expert_rows; int x_slot_stride; int y_slot_stride;
  // RMSNorm hand-off between consecutive batch-1 Q4_K layers: the producer leaves per-work-group partials of
  // sum(y^2) (1024 floats) that the consumer sums instead of re-reducing its input.  Both optional.
  const float* ssq_in; float* ssq_out;
};
// norm_gain != null fuses RMSNorm(eps) of x into the staging; swiglu_half > 0 computes
// y[i] = up_i * silu(gate_i) from rows i and swiglu_half + i of the (single) matrix.
int launch_gemv_multi(const MultiGemv& m, const float* x, int n_b, float* y, int64_t y_stride, int act,
                      const float* residual, const float* norm_gain, float norm_eps, int swiglu_half);
bool gemv_hands_off_ssq(const cai_qw_s* w, int n_b);
bool gemv_fuses_swiglu(const cai_qw_s* w, int n_b, bool expert_bank);
int launch_dequant_rows(const cai_qw_s* w, int64_t row0, int64_t n_rows, float* out);
int launch_rmsnorm(const float* x, const float* gain, int n, int n_tokens, float eps, float* y);
int launch_rope(float* x, int n_heads, int head_dim, const int32_t* pos_dev, int pos_host, const float* theta, int n_tokens, int64_t token_stride);
int launch_swiglu(const float* x, int half, int n_tokens, float* y);
int launch_add(float* x, const float* y, int64_t n);
int launch_argmax(const float* x, int n, int n_rows, int32_t* out, float* scratch_v, int32_t* scratch_i);
int argmax_scratch_entries(int n, int n_rows);
int noalloc_setup(int device);   // resolves the device address of the fixed scratch array (cai_init, device current)
int launch_embed(const cai_qw_s* w, const int32_t* tokens_dev, int n_tokens, float* out);
int launch_router_topk(const float* logits, int n, int k, int renorm, int n_tokens, int32_t* expert_out, float* gate_out, float* probs_scratch);
// ... and the router's matrix-vector product, RMSNorm and selection in one launch (Q8_0 router rows, up to 64 experts)
bool router_fused_supported(const cai_qw_s* w, int k);
int launch_router_fused(const cai_qw_s* w, const float* x, int64_t x_stride, const float* gain, float eps, int k, int renorm, int n_tokens,
                        float* logits_out, int32_t* expert_out, float* gate_out, float* probs_scratch, unsigned* counters);   // counters: one per token, zero before the first launch (they wrap back to zero)
int launch_rmsnorm_strided(const float* x, const float* gain, int n, int n_tokens, float eps, float* y, int64_t x_stride, int64_t y_stride);
void decoder_adopt_weight(cai_decoder_s* d, cai_qw_s* w);   // the decoder destroys w with itself
int launch_rmsnorm_pair(float* x, const float* gain_a, int n_a, const float* gain_b, int n_b, int n_tokens, float eps, int64_t stride);
int launch_moe_combine(float* x, const float* part, const float* gate, int k, int n, int n_tokens);
// gathered down projection of one token's k experts and the mixture into x[dm] in one launch (Q8_0 bank, k <= 8; mid: [k][cols])
bool moe_down_mix_supported(const cai_qw_s* w, int dm, int k);
int launch_moe_down_mix(const cai_qw_s* w, int dm, const float* mid, const int32_t* experts, const float* gates, int k, float* x);
int launch_split_blocks(const uint8_t* raw, int block_bytes, int64_t n_blocks, uint8_t* qs, uint16_t* d);
int launch_split_q6k(const uint8_t* raw, int64_t n_blocks, uint8_t* rec, uint8_t* sc, uint16_t* d);
// qkv: [n_seq][qkv_stride] rows [Q|K|V]; theta != null applies interleaved RoPE to Q and K first.  pos_dev[s] is
// both the rotary position and the cache slot the new K,V row goes to; the live range is [.., pos_dev[s]].
// Activation row s uses cache sequence seq0 + s.  prompt_rows != 0: the n_seq rows are consecutive tokens of ONE
// sequence (seq0): their K,V rows are appended first, then every row attends up to its own position; prompt_part must
// hold n_seq * q_heads * n_splits * (head_dim + 2) floats.  1 = a prompt chunk (eight rows or more of a 128-wide cache go to the
// matrix-core kernel, which may grow its operand planes); 2 = a window step inside a captured graph (decode kernels only,
// nothing is allocated).
int launch_attn_step(cai_kv_s* kv, int layer, float* qkv, int64_t qkv_stride, int n_seq, int q_heads, int window,
                     float softcap, const float* theta, const int32_t* pos_dev, float* out, int64_t out_stride, int seq0,
                     int prompt_rows = 0, float* prompt_part = nullptr,
                     const float* qn_gain = nullptr, const float* kn_gain = nullptr, float qk_eps = 0.0f);   // full-width q / k RMSNorm done on the way (null: none)
int kv_alloc(cai_kv_s* kv, int n_seq, int n_layers, int kv_heads, int head_dim, int max_ctx, int dtype);
void kv_free(cai_kv_s* kv);
int kv_set_eviction(cai_kv_s* kv, int sinks, int recent);
int kv_snapshot(cai_kv_s* kv, int seq, cai_kv_snap_s** out);
int kv_restore(cai_kv_s* kv, int seq, const cai_kv_snap_s* snap);
int kv_fork(cai_kv_s* kv, int src, int dst);
// Slice geometry by the rows in use, not by max_ctx: a session created for 32768 rows that holds 600 would otherwise cut them
// into 3 slices of 256 (12 busy work-groups on the 7B shape; 463 against 597 tok/s).  Lengths fall into buckets of 1024 * 2^b rows
// (a captured graph holds its launch geometry, so the decoder keeps one graph per bucket); kv_bucket_rows gives the bucket's
// upper bound for a needed row count (max_ctx for the last one), kv_geometry the slice length and count for it.
int kv_bucket_rows(const cai_kv_s* kv, int needed_rows);
bool attn_prompt_is_flash(const cai_kv_s* kv, int n);
void kv_geometry(const cai_kv_s* kv, int rows, int* split_len, int* n_splits);
// multi-token linear layer (matrix cores for Q4_K, small-batch kernel otherwise); gain != null fuses RMSNorm
int prefill_linear(const cai_qw_s* w, const float* x, int64_t x_stride, const float* gain, float eps, int n_tok,
                   float* y, int64_t y_stride, const float* residual);
bool gemm_mfma_supported(const cai_qw_s* w);   // many-token (prompt) matrix-core kernel of the super-block types (Q4_K, Q6_K)
bool gemm_blk_supported(const cai_qw_s* w);    // many-token (prompt) matrix-core kernel of the 32-weight block types (Q8_0, Q4_0)
inline bool prompt_gemm_supported(const cai_qw_s* w) { return gemm_mfma_supported(w) || gemm_blk_supported(w); }
int launch_gemm_blk(const cai_qw_s* w, const _Float16* xhi, const _Float16* xlo, const float* sinv, int n_tok, float* y, int64_t y_stride, const float* residual);
// mixture-of-experts prompt: slots (token * top_k + rank) grouped by expert, then one launch over the bank per projection
int moe_group_max_tiles(int n_slots, int n_experts);
int launch_moe_group(const int32_t* expert, int n_slots, int n_experts, int32_t* perm, int32_t* tile_tab);
int launch_gemm_blk_grouped(const cai_qw_s* bank, int64_t expert_rows, const _Float16* xhi, const _Float16* xlo, const float* sinv, int x_div,
                            int n_slots, int n_experts, const int32_t* perm, const int32_t* tile_tab, float* y, int64_t y_stride);
void prefill_planes(const _Float16** hi, const _Float16** lo, const float** sinv);   // what the last prefill_prep filled
int  prompt_route(const cai_qw_s* w, int n_tok);   // 0 matrix-vector passes, 1 small-batch kernel, 2 prompt kernel
bool nb_supported(const cai_qw_s* w);          // 2..8-token matrix-core kernel
// split pre-pass / product form: prep once, then any number of matrices of that width
// small-batch (<= 8 tokens per pass) matrix-core path: planes <- activations, partials <- product, consumer sums the slices
int nb_ws_generation();                                        // changes whenever its workspace buffers are reallocated
void nb_release();                                             // frees the small-batch workspace (cai_shutdown)
void prefill_release();                                        // frees the prompt workspace (cai_shutdown)
int nb_reserve(int k_max, size_t part_floats);                 // never inside a stream capture
// small-batch Q4_K products with the activations held in registers (cai_gemm_ra.hip): one launch per linear layer
bool ra_supported(const cai_qw_s* const* ws, int n_w, bool normed, int swiglu_half);
size_t ra_part_floats(int64_t rows, int64_t cols);
int ra_reserve(size_t part_floats);                            // never inside a stream capture
int ra_ws_generation();
void ra_release();
int ra_gemm(const cai_qw_s* const* ws, const int* y_off, int n_w, int n_tok, const float* x, int64_t x_stride, const float* gain, float eps,
            int swiglu_half, float* y, int64_t y_stride, const float* residual);
int nb_max_slices(int cols);
int nb_prep_plain(const float* x, int64_t x_stride, const float* gain, float eps, int K, int n_tok);
int nb_prep_residual(float* res, int64_t res_stride, const float* gain, float eps, int K, int n_tok);   // res += last product
int nb_prep_swiglu(int half, int n_tok);                       // planes <- SwiGLU(last product)
int nb_gemm(const cai_qw_s* const* ws, const int* y_off, int n_w, int n_tok);
int nb_reduce(float* y, int64_t y_stride, const float* residual);
int nb_linear(const cai_qw_s* w, const float* x, int64_t x_stride, const float* gain, float eps, int n_tok, float* y, int64_t y_stride, const float* residual);
int prefill_prep(const float* x, int64_t x_stride, const float* gain, float eps, int K, int n_tok);
int prefill_reserve_rows(int n_tok, int K);   // sizes the shared activation planes ahead of the first prefill_prep
int prefill_prep_swiglu(const float* gu, int64_t gu_stride, int half, int n_tok);   // planes <- up * silu(gate)
int prefill_gemm(const cai_qw_s* w, int n_tok, float* y, int64_t y_stride, const float* residual);
int prefill_gemm_multi(const cai_qw_s* const* ws, const int* y_off, int n_w, int n_tok, float* y, int64_t y_stride);
bool gemm_q4k_multi_supported(const cai_qw_s* const* ws, int n_w);
bool gemm_blk_multi_supported(const cai_qw_s* const* ws, int n_w);
int launch_gemm_blk_multi(const cai_qw_s* const* ws, const int* y_off, int n_w, const _Float16* xhi, const _Float16* xlo, const float* sinv,
                          int n_tok, float* y, int64_t y_stride);
bool prefill_multi_supported(const cai_qw_s* const* ws, int n_w);   // one launch of a prompt kernel takes these matrices together
int launch_gemm_q4k_multi(const cai_qw_s* const* ws, const int* y_off, int n_w, const _Float16* xhi, const _Float16* xlo, const _Float16* sxhi,
                          const _Float16* sxlo, const float* sinv, int n_tok, float* y, int64_t y_stride, const float* residual, int swiglu_half);
bool prefill_gemm_swiglu_supported(const cai_qw_s* w, int n_tok);
int prefill_gemm_swiglu(const cai_qw_s* w, int n_tok, float* y, int64_t y_stride);   // y[t][i] = up_i * silu(gate_i), on the planes of the last prefill_prep

void rope_thetas(float base, int head_dim, std::vector<float>& out);
int  rope_thetas_scaled(float base, int head_dim, int mode, float factor, int original_ctx, float low_freq_factor, float high_freq_factor, std::vector<float>& out);

// softmax -> history penalty -> temperature -> the m most probable tokens (descending) of a device-resident logits row;
// history and results are host arrays
int run_candidates(const float* logits_dev, int n, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                   float repetition, float frequency, float presence, float temperature, int m,
                   int32_t* tokens_out, float* probs_out, int* count_out);

}  // namespace cai
