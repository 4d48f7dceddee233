// Step-resident decoder: one token per sequence per step, every activation stays in HBM/L2 for the whole
// step, the launch sequence is captured once per batch width into a HIP graph and replayed.
//
// Graph order follows the reference importer (neural/neuralpretrained.pas:16384-16882) and one
// StepForward (neural/neuraldecode.pas:5696-5712):
//   Embedding -> per block { TokenRMSNorm -> q,k,v (+bias) -> [full-width q/k RMSNorm] -> RoPE -> FusedSDPA
//   (append + cached GQA) -> o-proj -> Sum -> TokenRMSNorm -> gate|up -> SwiGLU -> down -> Sum }
//   -> final TokenRMSNorm -> vocab projection -> ArgMaxRow.
// MoE blocks (neural/neuralpretrained.pas:15331-15388): router -> softmax -> top-k gate -> expert banks.
#include "cai_internal.hpp"

#include <algorithm>
#include <map>

struct cai_decoder_s {
  cai_decoder_config cfg{};
  struct Layer { cai_qw_s* w[9] = {nullptr}; float* v[5] = {nullptr}; };
  std::vector<Layer> layers;
  cai_qw_s* embed = nullptr; cai_qw_s* head = nullptr;
  float* final_norm = nullptr;
  float* theta = nullptr;
  cai_kv_s kv;
  float *x = nullptr, *qkv = nullptr, *att = nullptr, *gu = nullptr, *mid = nullptr, *logits = nullptr;
  float *router_logits = nullptr, *router_probs = nullptr, *moe_gate = nullptr, *moe_part = nullptr;
  int32_t* moe_expert = nullptr;
  float* am_v = nullptr; int32_t* am_i = nullptr;   // arg-max slice winners
  float* ssq = nullptr;                              // 2 x 1024 sum-of-squares partials (RMSNorm hand-off)
  // prompt ingestion (multi-token) buffers, allocated at the first prefill: rows of up to pf_cap tokens
  int pf_cap = 0;
  float *px = nullptr, *pqkv = nullptr, *patt = nullptr, *pgu = nullptr, *pmid = nullptr, *ppart = nullptr;
  size_t ppart_elems = 0;                            // (per row, query head and cache slice: sized for the length bucket in use)
  int ppart_rows = 1;                                // prompt rows per attention launch that ppart holds (ensure_ppart)
  int32_t* ptokpos = nullptr;                        // [2][pf_cap]: tokens, positions
  // mixture-of-experts prompt: per chunk the router outputs, the slots grouped by expert and the per-slot activations
  float *pm_logits = nullptr, *pm_probs = nullptr, *pm_gate = nullptr, *pm_gu = nullptr, *pm_part = nullptr;
  int32_t *pm_expert = nullptr, *pm_perm = nullptr, *pm_tiles = nullptr;
  int32_t *d_tokens = nullptr, *d_pos = nullptr, *d_argmax = nullptr, *d_gen = nullptr, *d_gen_idx = nullptr;
  int32_t* h_io = nullptr;   // pinned: tokens[8] pos[8] argmax[8] generated-so-far[8]
  // captured launch sequences of sequence 0, keyed by kind (0 batched step, 1 window step of one sequence, 2 greedy steps with
  // their hand-overs), width (rows or steps) and the cache-length bucket whose slice geometry the attention launches hold
  std::map<int, hipGraphExec_t> graphs;
  static int graph_key(int kind, int width, int bucket_rows) { return (kind << 28) | (width << 20) | (bucket_rows >> 8); }
  float* wpart = nullptr; size_t wpart_elems = 0;     // attention slice results of a window's rows (sized at the first window step)
  bool use_graph = true;
  int ws_generation = -1;         // activation-workspace generation the captured batch graphs were built against
  std::vector<cai_qw_s*> owned;   // weights created by a loader on the decoder's behalf, destroyed with it
  bool cache_lost = false;        // a change of cache type ran out of memory twice: the session has no K,V storage
  int qw() const { return cfg.n_q_heads * cfg.head_dim; }
  int kw() const { return cfg.n_kv_heads * cfg.head_dim; }
};

namespace cai {

// Greedy hand-over between two steps on the device: the arg-max becomes the next input token, the position advances, and
// the token is appended to the generated list (its length lives on the device, so the launch has no per-step argument and
// a captured graph of several steps replays).
__global__ void advance_kernel(int32_t* tokens, int32_t* pos, const int32_t* argmax, int32_t* gen_out, int32_t* gen_idx)
{
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    const int32_t t = argmax[0];
    const int idx = gen_idx[0];
    gen_out[idx] = t; gen_idx[0] = idx + 1; tokens[0] = t; pos[0] += 1;
  }
}
constexpr int GEN_UNROLL = 8;     // decode steps per launch of the long generation graph

static void invalidate_graphs(cai_decoder_s* d)
{
  for (auto& kvp : d->graphs) if (kvp.second) (void)hipGraphExecDestroy(kvp.second);
  d->graphs.clear();
}

static int check_ready(cai_decoder_s* d)
{
  const cai_decoder_config& c = d->cfg;
  if (d->cache_lost) return set_error(CAI_ERR_STATE, "decoder: the K,V cache was lost when cai_decoder_set_kv_dtype ran out of device memory; destroy the session");
  if (!d->embed) return set_error(CAI_ERR_STATE, "decoder: embedding weight not set");
  if (!d->final_norm) return set_error(CAI_ERR_STATE, "decoder: final norm gain not set");
  for (int l = 0; l < c.n_layers; l++) {
    const auto& L = d->layers[l];
    const int need_w[] = {CAI_W_Q, CAI_W_K, CAI_W_V, CAI_W_O, CAI_W_GATEUP, CAI_W_DOWN};
    for (int s : need_w) if (!L.w[s]) return set_error(CAI_ERR_STATE, "decoder: layer %d weight slot %d not set", l, s);
    if (c.n_experts > 0 && !L.w[CAI_W_ROUTER]) return set_error(CAI_ERR_STATE, "decoder: layer %d router not set", l);
    if (!L.v[CAI_V_ATTN_NORM] || !L.v[CAI_V_MLP_NORM]) return set_error(CAI_ERR_STATE, "decoder: layer %d norm gains not set", l);
    if (c.qk_norm_full && (!L.v[CAI_V_Q_NORM] || !L.v[CAI_V_K_NORM])) return set_error(CAI_ERR_STATE, "decoder: layer %d q/k norm gains not set", l);
  }
  return CAI_OK;
}


// Expert half of a block for n_b (<= 8) activation rows x[b][d_model], in place: router -> soft-max -> top-k
// gates -> gathered gate|up (RMSNorm and SwiGLU fused) -> gathered down -> gate-weighted mixture added to the row
// (neural/neuralpretrained.pas:15331-15388; neural/neural.cl:2689-2752).
static int moe_ffn_rows(cai_decoder_s* d, const cai_decoder_s::Layer& L, float* x, int n_b)
{
  const cai_decoder_config& c = d->cfg;
  const int dm = c.d_model, I = c.ffn;
  int rc;
  const int E = c.n_experts, K = c.top_k;
  if (router_fused_supported(L.w[CAI_W_ROUTER], K) && L.w[CAI_W_ROUTER]->rows == E && dm % 4 == 0) {
    if ((rc = launch_router_fused(L.w[CAI_W_ROUTER], x, dm, L.v[CAI_V_MLP_NORM], c.eps, K, c.norm_topk, n_b, d->router_logits, d->moe_expert, d->moe_gate, d->router_probs, reinterpret_cast<unsigned*>(d->moe_expert + 8 * K)))) return rc;
  } else {
    MultiGemv r{}; r.n = 1; r.w[0] = L.w[CAI_W_ROUTER]; r.rows[0] = E;
    if ((rc = launch_gemv_multi(r, x, n_b, d->router_logits, E, CAI_ACT_NONE, nullptr, L.v[CAI_V_MLP_NORM], c.eps, 0))) return rc;
    if ((rc = launch_router_topk(d->router_logits, E, K, c.norm_topk, n_b, d->moe_expert, d->moe_gate, d->router_probs))) return rc;
  }
  for (int b = 0; b < n_b; b++) {
    MultiGemv g{}; g.n = 1; g.w[0] = L.w[CAI_W_GATEUP]; g.rows[0] = 2 * I;
    g.slot_expert = d->moe_expert + b * K; g.n_slots = K; g.expert_rows = 2 * I; g.x_slot_stride = 0;
    const float* xb = x + (int64_t)b * dm;
    if (gemv_fuses_swiglu(g.w[0], 1, true)) {
      g.y_slot_stride = I;
      if ((rc = launch_gemv_multi(g, xb, 1, d->mid, I, CAI_ACT_NONE, nullptr, L.v[CAI_V_MLP_NORM], c.eps, I))) return rc;
    } else {
      g.y_slot_stride = 2 * I;
      if ((rc = launch_gemv_multi(g, xb, 1, d->gu, 2 * I, CAI_ACT_NONE, nullptr, L.v[CAI_V_MLP_NORM], c.eps, 0))) return rc;
      launch_swiglu(d->gu, I, K, d->mid);
    }
    if (moe_down_mix_supported(L.w[CAI_W_DOWN], dm, K) && I % 4 == 0) {
      if ((rc = launch_moe_down_mix(L.w[CAI_W_DOWN], dm, d->mid, d->moe_expert + b * K, d->moe_gate + b * K, K, x + (int64_t)b * dm))) return rc;
      continue;
    }
    MultiGemv dn{}; dn.n = 1; dn.w[0] = L.w[CAI_W_DOWN]; dn.rows[0] = dm;
    dn.slot_expert = d->moe_expert + b * K; dn.n_slots = K; dn.expert_rows = dm; dn.x_slot_stride = I; dn.y_slot_stride = dm;
    if ((rc = launch_gemv_multi(dn, d->mid, 1, d->moe_part, dm, CAI_ACT_NONE, nullptr, nullptr, 0.0f, 0))) return rc;
    launch_moe_combine(x + (int64_t)b * dm, d->moe_part, d->moe_gate + b * K, K, dm, 1);
  }
  return CAI_OK;
}

// Enqueues one whole step for activation rows 0..n_b-1 mapped to cache sequences seq0..seq0+n_b-1.
// `classes`: bit i set = launch kernel class i (0 embedding, 1 q|k|v, 2 attention, 3 o, 4 gate|up + SwiGLU, 5 down, 6 vocabulary
// projection, 7 arg-max).  Everything but the per-class timing of cai_decoder_profile passes all bits.
// `window`: the rows are n_b CONSECUTIVE tokens of the one sequence seq0 (the width-K window of a speculative verify step,
// neural/neuraldecode.pas:1151-1183): row r is rotated to and appended at position pos[r] and attends to the rows before it.
static int enqueue_step(cai_decoder_s* d, int n_b, int seq0, unsigned classes = ~0u, bool window = false)
{
  const cai_decoder_config& c = d->cfg;
  const int dm = c.d_model, qw = d->qw(), kw = d->kw(), I = c.ffn, qkvw = qw + 2 * kw;
  int rc;
  int& tl_cls = ctx().tl.cls;    // class of the launches that follow (timeline records)
  tl_cls = 0;
  if ((classes & 1u) && (rc = launch_embed(d->embed, d->d_tokens, n_b, d->x))) return rc;
  float* ssq_o = d->ssq;          // written by the o-projection, read by gate|up
  float* ssq_d = d->ssq + 1024;   // written by the down projection, read by the next block's q|k|v
  bool have_ssq_d = false;
  bool down_pending = false;      // small-batch path: the last down product has not been added to x yet
  // 2..8 sequences on block-quantized weights: every linear layer goes to the matrix cores (weights streamed once for the batch)
  auto mma_layer = [&](const cai_decoder_s::Layer& L) {
    if (n_b < 2 || c.n_experts > 0) return false;
    const int slots[6] = {CAI_W_Q, CAI_W_K, CAI_W_V, CAI_W_O, CAI_W_GATEUP, CAI_W_DOWN};
    for (int sl : slots) if (!nb_supported(L.w[sl]) || L.w[sl]->qtype == CAI_I8ROW) return false;   // (per-row int8 products need the plain reduction for their row scale)
    return true;
  };
  // ... and when all six are Q4_K of widths the register-resident form takes, a linear layer is ONE launch: activations
  // quantised by the product itself, norm factor, bias, residual and SwiGLU in its epilogue (CAIHIP_SMALL_BATCH_PLANES=1
  // keeps the form with activation planes and slice partials)
  static const bool ra_on = []() { const char* e = getenv("CAIHIP_SMALL_BATCH_PLANES"); return !(e && e[0] == '1'); }();
  auto ra_layer = [&](const cai_decoder_s::Layer& L) {
    if (!ra_on || n_b < 2 || n_b > 8 || c.n_experts > 0) return false;
    const cai_qw_s* qkv3[3] = {L.w[CAI_W_Q], L.w[CAI_W_K], L.w[CAI_W_V]};
    const cai_qw_s* wo = L.w[CAI_W_O]; const cai_qw_s* wgu = L.w[CAI_W_GATEUP]; const cai_qw_s* wdn = L.w[CAI_W_DOWN];
    return ra_supported(qkv3, 3, true, 0) && ra_supported(&wo, 1, false, 0) && ra_supported(&wgu, 1, true, I) && ra_supported(&wdn, 1, false, 0);
  };
  for (int l = 0; l < c.n_layers; l++) {
    auto& L = d->layers[l];
    if (ra_layer(L)) {
      if (down_pending) { if ((rc = nb_prep_residual(d->x, dm, nullptr, 0.0f, dm, n_b))) return rc; down_pending = false; }
      const cai_qw_s* qkv3[3] = {L.w[CAI_W_Q], L.w[CAI_W_K], L.w[CAI_W_V]}; const int off3[3] = {0, qw, qw + kw};
      tl_cls = 1;
      if ((rc = ra_gemm(qkv3, off3, 3, n_b, d->x, dm, L.v[CAI_V_ATTN_NORM], c.eps, 0, d->qkv, qkvw, nullptr))) return rc;
      tl_cls = 2;
      if ((rc = launch_attn_step(&d->kv, l, d->qkv, qkvw, n_b, c.n_q_heads, c.window, 0.0f, d->theta, d->d_pos, d->att, qw, seq0, window ? 2 : 0, window ? d->wpart : nullptr,
                                 c.qk_norm_full ? L.v[CAI_V_Q_NORM] : nullptr, c.qk_norm_full ? L.v[CAI_V_K_NORM] : nullptr, c.eps))) return rc;
      const int zero = 0;
      const cai_qw_s* wo = L.w[CAI_W_O]; const cai_qw_s* wgu = L.w[CAI_W_GATEUP]; const cai_qw_s* wdn = L.w[CAI_W_DOWN];
      tl_cls = 3;
      if ((rc = ra_gemm(&wo, &zero, 1, n_b, d->att, qw, nullptr, 0.0f, 0, d->x, dm, d->x))) return rc;
      tl_cls = 4;
      if ((rc = ra_gemm(&wgu, &zero, 1, n_b, d->x, dm, L.v[CAI_V_MLP_NORM], c.eps, I, d->mid, I, nullptr))) return rc;
      tl_cls = 5;
      if ((rc = ra_gemm(&wdn, &zero, 1, n_b, d->mid, I, nullptr, 0.0f, 0, d->x, dm, d->x))) return rc;
      have_ssq_d = false;
      continue;
    }
    if (mma_layer(L)) {
      // the down product of the previous block is still in slices: the pre-pass adds it to the residual stream
      if (down_pending) rc = nb_prep_residual(d->x, dm, L.v[CAI_V_ATTN_NORM], c.eps, dm, n_b);
      else rc = nb_prep_plain(d->x, dm, L.v[CAI_V_ATTN_NORM], c.eps, dm, n_b);
      if (rc) return rc;
      down_pending = false;
      {
        const cai_qw_s* qkv3[3] = {L.w[CAI_W_Q], L.w[CAI_W_K], L.w[CAI_W_V]}; const int off3[3] = {0, qw, qw + kw};
        if ((rc = nb_gemm(qkv3, off3, 3, n_b)) || (rc = nb_reduce(d->qkv, qkvw, nullptr))) return rc;
      }
      if ((rc = launch_attn_step(&d->kv, l, d->qkv, qkvw, n_b, c.n_q_heads, c.window, 0.0f, d->theta, d->d_pos, d->att, qw, seq0, window ? 2 : 0, window ? d->wpart : nullptr,
                                 c.qk_norm_full ? L.v[CAI_V_Q_NORM] : nullptr, c.qk_norm_full ? L.v[CAI_V_K_NORM] : nullptr, c.eps))) return rc;
      const int zero = 0;
      const cai_qw_s* wo = L.w[CAI_W_O]; const cai_qw_s* wgu = L.w[CAI_W_GATEUP]; const cai_qw_s* wdn = L.w[CAI_W_DOWN];
      if ((rc = nb_prep_plain(d->att, qw, nullptr, 0.0f, qw, n_b)) || (rc = nb_gemm(&wo, &zero, 1, n_b))) return rc;
      if ((rc = nb_prep_residual(d->x, dm, L.v[CAI_V_MLP_NORM], c.eps, dm, n_b)) || (rc = nb_gemm(&wgu, &zero, 1, n_b))) return rc;
      if ((rc = nb_prep_swiglu(I, n_b)) || (rc = nb_gemm(&wdn, &zero, 1, n_b))) return rc;
      down_pending = true;
      have_ssq_d = false;
      continue;
    }
    if (down_pending) { if ((rc = nb_prep_residual(d->x, dm, nullptr, 0.0f, dm, n_b))) return rc; down_pending = false; }
    // --- attention half ---
    tl_cls = 1;
    if (classes & 2u) {
      MultiGemv m{}; m.n = 3;
      const int slots[3] = {CAI_W_Q, CAI_W_K, CAI_W_V}; const int offs[3] = {0, qw, qw + kw};
      bool same = true;
      for (int i = 0; i < 3; i++) {
        m.w[i] = L.w[slots[i]]; m.row0[i] = 0; m.rows[i] = m.w[i]->rows; m.y_off[i] = offs[i];
        same = same && m.w[i]->qtype == m.w[0]->qtype;
      }
      if (same && have_ssq_d && gemv_hands_off_ssq(m.w[0], n_b)) m.ssq_in = ssq_d;
      if (same) {
        if ((rc = launch_gemv_multi(m, d->x, n_b, d->qkv, qkvw, CAI_ACT_NONE, nullptr, L.v[CAI_V_ATTN_NORM], c.eps, 0))) return rc;
      } else {
        bool done[3] = {false, false, false};       // one launch per weight type (attn_v of a mixed file differs from attn_q, attn_k)
        for (int i0 = 0; i0 < 3; i0++) {
          if (done[i0]) continue;
          MultiGemv grp{};
          for (int i = i0; i < 3; i++) {
            if (m.w[i]->qtype != m.w[i0]->qtype) continue;
            done[i] = true;
            grp.w[grp.n] = m.w[i]; grp.rows[grp.n] = m.rows[i]; grp.y_off[grp.n] = offs[i]; grp.n++;
          }
          if ((rc = launch_gemv_multi(grp, d->x, n_b, d->qkv, qkvw, CAI_ACT_NONE, nullptr, L.v[CAI_V_ATTN_NORM], c.eps, 0))) return rc;
        }
      }
    }
    tl_cls = 2;
    if ((classes & 4u) &&
        (rc = launch_attn_step(&d->kv, l, d->qkv, qkvw, n_b, c.n_q_heads, c.window, 0.0f, d->theta, d->d_pos, d->att, qw, seq0, window ? 2 : 0, window ? d->wpart : nullptr,
                               c.qk_norm_full ? L.v[CAI_V_Q_NORM] : nullptr, c.qk_norm_full ? L.v[CAI_V_K_NORM] : nullptr, c.eps))) return rc;
    const bool o_hands = gemv_hands_off_ssq(L.w[CAI_W_O], n_b);
    tl_cls = 3;
    if (classes & 8u) {
      MultiGemv m{}; m.n = 1; m.w[0] = L.w[CAI_W_O]; m.rows[0] = dm;
      if (o_hands) m.ssq_out = ssq_o;
      if ((rc = launch_gemv_multi(m, d->att, n_b, d->x, dm, CAI_ACT_NONE, d->x, nullptr, 0.0f, 0))) return rc;
    }
    have_ssq_d = false;
    // --- feed-forward half ---
    tl_cls = 4;
    if (c.n_experts == 0) {
      MultiGemv m{}; m.n = 1; m.w[0] = L.w[CAI_W_GATEUP]; m.rows[0] = 2 * I;
      if (o_hands && gemv_hands_off_ssq(m.w[0], n_b)) m.ssq_in = ssq_o;
      if (!(classes & 16u)) {
      } else if (gemv_fuses_swiglu(m.w[0], n_b, false)) {
        if ((rc = launch_gemv_multi(m, d->x, n_b, d->mid, I, CAI_ACT_NONE, nullptr, L.v[CAI_V_MLP_NORM], c.eps, I))) return rc;
      } else {
        if ((rc = launch_gemv_multi(m, d->x, n_b, d->gu, 2 * I, CAI_ACT_NONE, nullptr, L.v[CAI_V_MLP_NORM], c.eps, 0))) return rc;
        launch_swiglu(d->gu, I, n_b, d->mid);
      }
      have_ssq_d = gemv_hands_off_ssq(L.w[CAI_W_DOWN], n_b);
      tl_cls = 5;
      if (classes & 32u) {
        MultiGemv dn{}; dn.n = 1; dn.w[0] = L.w[CAI_W_DOWN]; dn.rows[0] = dm;
        if (have_ssq_d) dn.ssq_out = ssq_d;
        if ((rc = launch_gemv_multi(dn, d->mid, n_b, d->x, dm, CAI_ACT_NONE, d->x, nullptr, 0.0f, 0))) return rc;
      }
    } else {
      if ((classes & 48u) && (rc = moe_ffn_rows(d, L, d->x, n_b))) return rc;
    }
  }
  tl_cls = 6;
  if (classes & 64u) {
    cai_qw_s* hw = d->head ? d->head : d->embed;   // tied head (neural/neuralpretrained.pas:15555-)
    if (n_b >= 2 && nb_supported(hw)) {
      const int zero = 0; const cai_qw_s* hwc = hw;
      if (down_pending) rc = nb_prep_residual(d->x, dm, d->final_norm, c.eps, dm, n_b);
      else rc = nb_prep_plain(d->x, dm, d->final_norm, c.eps, dm, n_b);
      if (rc || (rc = nb_gemm(&hwc, &zero, 1, n_b)) || (rc = nb_reduce(d->logits, c.vocab, nullptr))) return rc;
      launch_argmax(d->logits, c.vocab, n_b, d->d_argmax, d->am_v, d->am_i);
      return CAI_OK;
    }
    if (down_pending) { if ((rc = nb_prep_residual(d->x, dm, nullptr, 0.0f, dm, n_b))) return rc; down_pending = false; }
    MultiGemv m{}; m.n = 1; m.w[0] = hw; m.rows[0] = c.vocab;
    if (have_ssq_d && gemv_hands_off_ssq(hw, n_b)) m.ssq_in = ssq_d;
    if ((rc = launch_gemv_multi(m, d->x, n_b, d->logits, c.vocab, CAI_ACT_NONE, nullptr, d->final_norm, c.eps, 0))) return rc;
  }
  if (classes & 128u) launch_argmax(d->logits, c.vocab, n_b, d->d_argmax, d->am_v, d->am_i);
  return CAI_OK;
}


// Multi-token prompt ingestion of one chunk (n <= pf_cap tokens of sequence `seq` at positions pos0..): every linear
// layer runs once for the whole chunk (matrix cores for Q4_K), K,V rows are appended, then each token attends up to
// its own position.  Equals n sequential steps (the reference's prefill, neural/neuralchatengine.pas:1466-1470).
static void free_moe_prompt(cai_decoder_s* d)
{
  void* q[] = {d->pm_logits, d->pm_probs, d->pm_gate, d->pm_gu, d->pm_part, d->pm_expert, d->pm_perm, d->pm_tiles};
  for (void* v : q) if (v) (void)hipFree(v);
  d->pm_logits = d->pm_probs = d->pm_gate = d->pm_gu = d->pm_part = nullptr;
  d->pm_expert = d->pm_perm = d->pm_tiles = nullptr;
}

static int ensure_prefill_buffers(cai_decoder_s* d, int n)
{
  if (d->pf_cap >= n) return CAI_OK;
  const cai_decoder_config& c = d->cfg;
  const int cap = std::max(n, 128);
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  { float* pf[] = {d->px, d->pqkv, d->patt, d->pgu, d->pmid, d->ppart}; for (float* q : pf) if (q) (void)hipFree(q); }
  if (d->ptokpos) (void)hipFree(d->ptokpos);
  d->px = d->pqkv = d->patt = d->pgu = d->pmid = d->ppart = nullptr; d->ptokpos = nullptr; d->pf_cap = 0; d->ppart_elems = 0;
  free_moe_prompt(d);
  const size_t qkvw = d->qw() + 2 * d->kw();
  CAI_HIP(hipMalloc((void**)&d->px, (size_t)cap * c.d_model * 4));
  CAI_HIP(hipMalloc((void**)&d->pqkv, (size_t)cap * qkvw * 4));
  CAI_HIP(hipMalloc((void**)&d->patt, (size_t)cap * d->qw() * 4));
  CAI_HIP(hipMalloc((void**)&d->pgu, (size_t)cap * 2 * c.ffn * 4));
  CAI_HIP(hipMalloc((void**)&d->pmid, (size_t)cap * c.ffn * 4));
  CAI_HIP(hipMalloc((void**)&d->ptokpos, (size_t)cap * 2 * sizeof(int32_t)));
  if (c.n_experts > 0 && c.n_experts <= 512) {
    const size_t E = c.n_experts, S = (size_t)cap * c.top_k;
    CAI_HIP(hipMalloc((void**)&d->pm_logits, (size_t)cap * E * 4)); CAI_HIP(hipMalloc((void**)&d->pm_probs, (size_t)cap * E * 4));
    CAI_HIP(hipMalloc((void**)&d->pm_gate, S * 4)); CAI_HIP(hipMalloc((void**)&d->pm_expert, S * 4)); CAI_HIP(hipMalloc((void**)&d->pm_perm, S * 4));
    CAI_HIP(hipMalloc((void**)&d->pm_tiles, (size_t)moe_group_max_tiles((int)S, c.n_experts) * 3 * 4));
    CAI_HIP(hipMalloc((void**)&d->pm_gu, S * 2 * c.ffn * 4)); CAI_HIP(hipMalloc((void**)&d->pm_part, S * c.d_model * 4));
  }
  d->pf_cap = cap;
  // the activation planes of the prompt products, sized once for the widest row (a mixture-of-experts chunk prepares one row per slot)
  const int plane_rows = c.n_experts > 0 ? cap * std::max(c.top_k, 1) : cap;
  return prefill_reserve_rows(plane_rows, std::max(std::max(c.d_model, d->qw()), c.ffn));
}

// Partial results of the prompt rows' attention when it runs on the decode kernels (rows x query heads x cache slices): sized
// for the slice count of the length bucket in use, so a session created for 131072 rows does not hold 512 slices' worth for a
// prompt at its start, and for at most 256 MiB: a chunk whose rows need more (512 slices x 32 heads x 66 floats are 4.3 MB
// per row) attends in groups of ppart_rows rows, one attention launch per group.  A chunk the matrix-core prompt kernel
// takes needs none.  Grown on demand; prompt passes are not captured, so the pointer may change between them.
// (CAIHIP_PROMPT_PART_KB: another bound, read once per process; the tests use it to reach the grouped form with small models)
static size_t ppart_bytes()
{
  static const size_t b = []() { const char* e = getenv("CAIHIP_PROMPT_PART_KB"); return e && atoll(e) > 0 ? (size_t)atoll(e) << 10 : (size_t)256 << 20; }();
  return b;
}
static int ensure_ppart(cai_decoder_s* d, int rows_needed, int n)
{
  if (attn_prompt_is_flash(&d->kv, n)) { d->ppart_rows = n; return CAI_OK; }
  int sl, ns;
  kv_geometry(&d->kv, kv_bucket_rows(&d->kv, rows_needed), &sl, &ns);
  const size_t per_row = (size_t)d->cfg.n_q_heads * ns * (d->cfg.head_dim + 2);
  const int rows = (int)std::max<size_t>(1, std::min<size_t>((size_t)n, ppart_bytes() / (per_row * sizeof(float))));
  const size_t need = per_row * rows;
  d->ppart_rows = rows;
  if (d->ppart && d->ppart_elems >= need) return CAI_OK;
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  if (d->ppart) { (void)hipFree(d->ppart); d->ppart = nullptr; }
  d->ppart_elems = 0;
  CAI_HIP(hipMalloc((void**)&d->ppart, need * sizeof(float)));
  d->ppart_elems = need;
  return CAI_OK;
}

static int linear_rows(const cai_qw_s* w, bool prepped, const float* x, int64_t x_stride, const float* gain, float eps, int n,
                       float* y, int64_t y_stride, const float* residual);

// Expert half of a block for a whole prompt chunk in px (n tokens), in place (neural/neuralpretrained.pas:15331-15388):
// router logits -> soft-max / top-k for every token -> the n * top_k slots grouped by expert -> gate|up over the bank in one
// launch -> SwiGLU -> down over the bank in one launch -> gate-weighted mixture added to each row.
static int moe_ffn_prompt(cai_decoder_s* d, const cai_decoder_s::Layer& L, int n)
{
  const cai_decoder_config& c = d->cfg;
  const int dm = c.d_model, I = c.ffn, E = c.n_experts, K = c.top_k, slots = n * K;
  int rc;
  if ((rc = linear_rows(L.w[CAI_W_ROUTER], false, d->px, dm, L.v[CAI_V_MLP_NORM], c.eps, n, d->pm_logits, E, nullptr))) return rc;
  if ((rc = launch_router_topk(d->pm_logits, E, K, c.norm_topk, n, d->pm_expert, d->pm_gate, d->pm_probs))) return rc;
  if ((rc = launch_moe_group(d->pm_expert, slots, E, d->pm_perm, d->pm_tiles))) return rc;
  const _Float16 *hi, *lo; const float* sinv;
  if ((rc = prefill_prep(d->px, dm, L.v[CAI_V_MLP_NORM], c.eps, dm, n))) return rc;
  prefill_planes(&hi, &lo, &sinv);
  if ((rc = launch_gemm_blk_grouped(L.w[CAI_W_GATEUP], 2 * (int64_t)I, hi, lo, sinv, K, slots, E, d->pm_perm, d->pm_tiles, d->pm_gu, 2 * I))) return rc;
  if ((rc = prefill_prep_swiglu(d->pm_gu, 2 * I, I, slots))) return rc;   // SwiGLU inside the pre-pass of the down projection
  prefill_planes(&hi, &lo, &sinv);
  if ((rc = launch_gemm_blk_grouped(L.w[CAI_W_DOWN], dm, hi, lo, sinv, 1, slots, E, d->pm_perm, d->pm_tiles, d->pm_part, dm))) return rc;
  return launch_moe_combine(d->px, d->pm_part, d->pm_gate, K, dm, n);
}

static int linear_rows(const cai_qw_s* w, bool prepped, const float* x, int64_t x_stride, const float* gain, float eps, int n,
                       float* y, int64_t y_stride, const float* residual)
{
  const int route = prompt_route(w, n);
  if (route == 1) return nb_linear(w, x, x_stride, gain, eps, n, y, y_stride, residual);
  if (route == 2) {
    int rc;
    if (!prepped && (rc = prefill_prep(x, x_stride, gain, eps, (int)w->cols, n))) return rc;
    return prefill_gemm(w, n, y, y_stride, residual);
  }
  return prefill_linear(w, x, x_stride, gain, eps, n, y, y_stride, residual);
}

static int enqueue_prefill_chunk(cai_decoder_s* d, int seq, int n)
{
  const cai_decoder_config& c = d->cfg;
  const int dm = c.d_model, qw = d->qw(), kw = d->kw(), I = c.ffn, qkvw = qw + 2 * kw;
  const int32_t* toks = d->ptokpos; const int32_t* poss = d->ptokpos + d->pf_cap;
  int rc;
  if ((rc = launch_embed(d->embed, toks, n, d->px))) return rc;
  for (int l = 0; l < c.n_layers; l++) {
    auto& L = d->layers[l];
    const cai_qw_s* wq = L.w[CAI_W_Q]; const cai_qw_s* wk = L.w[CAI_W_K]; const cai_qw_s* wv = L.w[CAI_W_V];
    const bool all_mfma = prompt_route(wq, n) == 2 && prompt_route(wk, n) == 2 && prompt_route(wv, n) == 2;   // one pre-pass serves q, k and v
    if (all_mfma && (rc = prefill_prep(d->px, dm, L.v[CAI_V_ATTN_NORM], c.eps, dm, n))) return rc;
    const cai_qw_s* qkv3[3] = {wq, wk, wv}; const int qkv_off[3] = {0, qw, qw + kw};
    if (all_mfma && prefill_multi_supported(qkv3, 3)) {   // one launch: the k and v projections alone leave half the chip idle
      if ((rc = prefill_gemm_multi(qkv3, qkv_off, 3, n, d->pqkv, qkvw))) return rc;
    } else if (all_mfma && prefill_multi_supported(qkv3, 2)) {   // attn_v of another type (a Q4_K_M file keeps some in Q6_K): q | k together
      if ((rc = prefill_gemm_multi(qkv3, qkv_off, 2, n, d->pqkv, qkvw))) return rc;
      if ((rc = linear_rows(wv, true, d->px, dm, L.v[CAI_V_ATTN_NORM], c.eps, n, d->pqkv + qw + kw, qkvw, nullptr))) return rc;
    } else {
      if ((rc = linear_rows(wq, all_mfma, d->px, dm, L.v[CAI_V_ATTN_NORM], c.eps, n, d->pqkv, qkvw, nullptr))) return rc;
      if ((rc = linear_rows(wk, all_mfma, d->px, dm, L.v[CAI_V_ATTN_NORM], c.eps, n, d->pqkv + qw, qkvw, nullptr))) return rc;
      if ((rc = linear_rows(wv, all_mfma, d->px, dm, L.v[CAI_V_ATTN_NORM], c.eps, n, d->pqkv + qw + kw, qkvw, nullptr))) return rc;
    }
    // (rows attend to the cache rows up to their own position, so a later group may be appended after an earlier one has attended)
    for (int r0 = 0; r0 < n; r0 += d->ppart_rows)
      if ((rc = launch_attn_step(&d->kv, l, d->pqkv + (int64_t)r0 * qkvw, qkvw, std::min(d->ppart_rows, n - r0), c.n_q_heads, c.window, 0.0f, d->theta,
                                 poss + r0, d->patt + (int64_t)r0 * qw, qw, seq, 1, d->ppart,
                                 c.qk_norm_full ? L.v[CAI_V_Q_NORM] : nullptr, c.qk_norm_full ? L.v[CAI_V_K_NORM] : nullptr, c.eps))) return rc;
    if ((rc = linear_rows(L.w[CAI_W_O], false, d->patt, qw, nullptr, 0.0f, n, d->px, dm, d->px))) return rc;
    if (c.n_experts > 0) {
      // experts differ from token to token.  A chunk of more than 16 tokens whose banks the block prompt kernel takes is
      // sorted by expert and runs each projection as ONE launch over the bank; otherwise the routed half runs on groups of
      // rows (one router / top-k launch per group, the gathered products per token)
      if (n > 16 && d->pm_gu && gemm_blk_supported(L.w[CAI_W_GATEUP]) && gemm_blk_supported(L.w[CAI_W_DOWN])) {
        if ((rc = moe_ffn_prompt(d, L, n))) return rc;
        continue;
      }
      const int grp = 8;
      for (int t0 = 0; t0 < n; t0 += grp)
        if ((rc = moe_ffn_rows(d, L, d->px + (int64_t)t0 * dm, std::min(grp, n - t0)))) return rc;
      continue;
    }
    if (prompt_route(L.w[CAI_W_GATEUP], n) == 2 && prefill_gemm_swiglu_supported(L.w[CAI_W_GATEUP], n)) {
      // SwiGLU in the epilogue of the gate|up product: a wave holds 32 up rows and their gate rows
      if ((rc = prefill_prep(d->px, dm, L.v[CAI_V_MLP_NORM], c.eps, dm, n))) return rc;
      if ((rc = prefill_gemm_swiglu(L.w[CAI_W_GATEUP], n, d->pmid, I))) return rc;
      if ((rc = linear_rows(L.w[CAI_W_DOWN], false, d->pmid, I, nullptr, 0.0f, n, d->px, dm, d->px))) return rc;
      continue;
    }
    if ((rc = linear_rows(L.w[CAI_W_GATEUP], false, d->px, dm, L.v[CAI_V_MLP_NORM], c.eps, n, d->pgu, 2 * I, nullptr))) return rc;
    if (prompt_route(L.w[CAI_W_DOWN], n) == 2) {   // SwiGLU inside the activation pre-pass of the down projection
      if ((rc = prefill_prep_swiglu(d->pgu, 2 * I, I, n))) return rc;
      if ((rc = linear_rows(L.w[CAI_W_DOWN], true, nullptr, I, nullptr, 0.0f, n, d->px, dm, d->px))) return rc;
    } else {
      launch_swiglu(d->pgu, I, n, d->pmid);
      if ((rc = linear_rows(L.w[CAI_W_DOWN], false, d->pmid, I, nullptr, 0.0f, n, d->px, dm, d->px))) return rc;
    }
  }
  return CAI_OK;
}

// `rows_needed`: cache rows the step's attention must cover (largest position + 1 over its rows)
static int run_step(cai_decoder_s* d, int n_b, int rows_needed, bool window = false, int seq0 = 0)
{
  Context& c = ctx();
  if (n_b >= 2) {   // the matrix-core path's activation workspace cannot grow inside a stream capture
    const cai_decoder_config& cf = d->cfg;
    const int dm = cf.d_model, qkvw = d->qw() + 2 * d->kw();
    const int kmax = std::max(std::max(dm, d->qw()), cf.ffn);
    auto al4 = [](int64_t v) { return (size_t)((v + 3) / 4 * 4); };
    size_t part = std::max(std::max((size_t)nb_max_slices(dm) * al4(qkvw), (size_t)nb_max_slices(d->qw()) * al4(dm)),
                           std::max((size_t)nb_max_slices(dm) * al4(2 * (int64_t)cf.ffn), (size_t)nb_max_slices(cf.ffn) * al4(dm)));
    part = std::max(part, (size_t)nb_max_slices(dm) * al4(cf.vocab)) * 8;
    int rc = nb_reserve(kmax, part); if (rc) return rc;
    if ((rc = ra_reserve(std::max(std::max(ra_part_floats(qkvw, dm), ra_part_floats(dm, d->qw())), std::max(ra_part_floats(2 * (int64_t)cf.ffn, dm), ra_part_floats(dm, cf.ffn)))))) return rc;   // (products of more than 16 super-blocks are sliced)
    const int gen = nb_ws_generation() + ra_ws_generation();      // (both only ever grow)
    if (d->ws_generation != gen) { invalidate_graphs(d); d->ws_generation = gen; }
  }
  const int bucket = kv_bucket_rows(&d->kv, rows_needed);
  d->kv.geo_rows = bucket;
  // (a captured graph holds the sequence index: only sequence 0 has one)
  if (!d->use_graph || seq0 != 0) { const int rc = enqueue_step(d, n_b, seq0, ~0u, window); if (rc) return rc; CAI_HIP(hipGetLastError()); return CAI_OK; }
  hipGraphExec_t& ge = d->graphs[cai_decoder_s::graph_key(window ? 1 : 0, n_b, bucket)];
  if (!ge) {
    hipGraph_t g = nullptr;
    CAI_HIP(hipStreamBeginCapture(c.stream, hipStreamCaptureModeThreadLocal));
    const int rc = enqueue_step(d, n_b, 0, ~0u, window);
    const hipError_t e = hipStreamEndCapture(c.stream, &g);
    if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
    if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture", __FILE__, __LINE__);
    const hipError_t e2 = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e2 != hipSuccess) return hip_fail(e2, "hipGraphInstantiate", __FILE__, __LINE__);
  }
  CAI_HIP(hipGraphLaunch(ge, c.stream));
  return CAI_OK;
}

// `steps` greedy batch-1 steps of sequence 0, each followed by the hand-over kernel, as ONE graph launch (steps = 1 or
// GEN_UNROLL): a launch per token costs the stream a gap between graphs and a separate hand-over launch.
static int run_gen_steps(cai_decoder_s* d, int steps, int rows_needed)
{
  Context& c = ctx();
  const int bucket = kv_bucket_rows(&d->kv, rows_needed);
  d->kv.geo_rows = bucket;
  auto body = [&]() {
    for (int u = 0; u < steps; u++) {
      const int rc = enqueue_step(d, 1, 0); if (rc) return rc;
      hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(64), 0, c.stream, d->d_tokens, d->d_pos, d->d_argmax, d->d_gen, d->d_gen_idx);
    }
    return (int)CAI_OK;
  };
  if (!d->use_graph) { const int rc = body(); if (rc) return rc; CAI_HIP(hipGetLastError()); return CAI_OK; }
  hipGraphExec_t& ge = d->graphs[cai_decoder_s::graph_key(2, steps, bucket)];
  if (!ge) {
    hipGraph_t g = nullptr;
    CAI_HIP(hipStreamBeginCapture(c.stream, hipStreamCaptureModeThreadLocal));
    const int rc = body();
    const hipError_t e = hipStreamEndCapture(c.stream, &g);
    if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
    if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture", __FILE__, __LINE__);
    const hipError_t e2 = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e2 != hipSuccess) return hip_fail(e2, "hipGraphInstantiate", __FILE__, __LINE__);
  }
  CAI_HIP(hipGraphLaunch(ge, c.stream));
  return CAI_OK;
}

// Scratch of a window step's attention: per (row, query head, cache slice) a partial result.
static int ensure_wpart(cai_decoder_s* d)
{
  const size_t need = (size_t)8 * d->kv.part_q_heads * d->kv.n_splits_alloc * (d->cfg.head_dim + 2);
  if (d->wpart && d->wpart_elems >= need) return CAI_OK;
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  if (d->wpart) { (void)hipFree(d->wpart); d->wpart = nullptr; }
  d->wpart_elems = 0;
  invalidate_graphs(d);                       // captured window steps hold the old pointer
  CAI_HIP(hipMalloc((void**)&d->wpart, need * sizeof(float)));
  d->wpart_elems = need;
  return CAI_OK;
}

// The most recent earlier occurrence of the context's last match_len tokens; the tokens that followed it (at most num_draft)
// are the draft (neural/neuraldecode.pas:7742-7765, PromptLookupDraft).  Returns the draft length (0: no match).
static int lookup_draft(const int32_t* ctx_tok, int n_ctx, int match_len, int num_draft, int32_t* draft)
{
  if (match_len < 1 || num_draft < 1 || n_ctx < match_len + 1) return 0;
  const int32_t* suffix = ctx_tok + n_ctx - match_len;
  for (int p = n_ctx - match_len - 1; p >= 0; p--) {      // start of a candidate; the suffix itself (p = n_ctx - match_len) is excluded
    bool same = true;
    for (int i = 0; i < match_len && same; i++) same = ctx_tok[p + i] == suffix[i];
    if (!same) continue;
    const int follow = std::min(n_ctx - (p + match_len), num_draft);
    for (int i = 0; i < follow; i++) draft[i] = ctx_tok[p + match_len + i];
    return follow;                                         // the most recent occurrence wins
  }
  return 0;
}

}  // namespace cai

using namespace cai;

extern "C" int cai_decoder_create(const cai_decoder_config* cfg, cai_decoder_t* out)
{
  CAI_ENTER();
  // (the shape is checked before the device is: a refused configuration is refused on any machine)
  CAI_REQUIRE(cfg && out, "cai_decoder_create: null argument");
  const cai_decoder_config& c = *cfg;
  CAI_REQUIRE(c.n_layers > 0 && c.d_model > 0 && c.n_q_heads > 0 && c.n_kv_heads > 0 && c.head_dim > 0 && c.ffn > 0 && c.vocab > 0 && c.max_ctx > 0,
              "cai_decoder_create: non-positive dimension");
  CAI_REQUIRE(c.n_q_heads % c.n_kv_heads == 0 && c.n_q_heads / c.n_kv_heads <= 8, "cai_decoder_create: %d query heads per %d KV heads unsupported", c.n_q_heads, c.n_kv_heads);
  CAI_REQUIRE(c.max_batch >= 1 && c.max_batch <= 8, "cai_decoder_create: max_batch %d outside 1..8", c.max_batch);
  CAI_REQUIRE(c.n_experts == 0 || (c.top_k >= 1 && c.top_k <= c.n_experts && c.top_k <= 64), "cai_decoder_create: top_k %d of %d experts", c.top_k, c.n_experts);
  // the router kernel ranks at most 512 experts; a larger bank would leave the gather's expert ids unwritten
  CAI_REQUIRE(c.n_experts >= 0 && c.n_experts <= 512, "cai_decoder_create: %d experts (supported: up to 512)", c.n_experts);
  CAI_READY();
  cai_decoder_s* d = new cai_decoder_s();
  d->cfg = c;
  d->layers.resize(c.n_layers);
  const int B = c.max_batch, qw = d->qw(), kw = d->kw();
  int rc = kv_alloc(&d->kv, B, c.n_layers, c.n_kv_heads, c.head_dim, c.max_ctx, c.kv_dtype);
  if (rc) { kv_free(&d->kv); delete d; return rc; }
  std::vector<float> th; rope_thetas(c.rope_theta, c.head_dim, th);
  auto alloc_f = [&](float** p, size_t n) { return hipMalloc((void**)p, n * sizeof(float)); };
  hipError_t e = alloc_f(&d->theta, th.size());
  const int K = std::max(c.top_k, 1);
  // activation rows: eight whatever max_batch is (a window step of ONE sequence is up to eight rows wide; only the K,V
  // cache grows with the number of sequences)
  constexpr int RB = 8;
  if (e == hipSuccess) e = alloc_f(&d->x, (size_t)RB * c.d_model);
  if (e == hipSuccess) e = alloc_f(&d->qkv, (size_t)RB * (qw + 2 * kw));
  if (e == hipSuccess) e = alloc_f(&d->att, (size_t)RB * qw);
  if (e == hipSuccess) e = alloc_f(&d->gu, (size_t)std::max(RB, K) * 2 * c.ffn);
  if (e == hipSuccess) e = alloc_f(&d->mid, (size_t)std::max(RB, K) * c.ffn);
  if (e == hipSuccess) e = alloc_f(&d->logits, (size_t)RB * c.vocab);
  if (c.n_experts > 0) {
    // (eight rows whatever the batch: a prompt routes its tokens in groups of eight)
    if (e == hipSuccess) e = alloc_f(&d->router_logits, (size_t)8 * c.n_experts);
    if (e == hipSuccess) e = alloc_f(&d->router_probs, (size_t)8 * c.n_experts);
    if (e == hipSuccess) e = alloc_f(&d->moe_gate, (size_t)8 * K);
    if (e == hipSuccess) e = alloc_f(&d->moe_part, (size_t)K * c.d_model);
    // (+ eight arrival counters of the one-launch router behind the selections: zero once, they wrap back to zero)
    if (e == hipSuccess) e = hipMalloc((void**)&d->moe_expert, (size_t)(8 * K + 8) * sizeof(int32_t));
    if (e == hipSuccess) e = hipMemsetAsync(d->moe_expert, 0, (size_t)(8 * K + 8) * sizeof(int32_t), ctx().stream);
  }
  const int ame = argmax_scratch_entries(c.vocab, RB);
  if (e == hipSuccess) e = alloc_f(&d->am_v, (size_t)ame);
  if (e == hipSuccess) e = hipMalloc((void**)&d->am_i, (size_t)ame * sizeof(int32_t));
  if (e == hipSuccess) e = alloc_f(&d->ssq, 2 * 1024);
  if (e == hipSuccess) e = hipMalloc((void**)&d->d_tokens, 4 * 8 * sizeof(int32_t));
  if (e == hipSuccess) e = hipMalloc((void**)&d->d_gen, (size_t)c.max_ctx * sizeof(int32_t));
  if (e == hipSuccess) e = hipHostMalloc((void**)&d->h_io, 4 * 8 * sizeof(int32_t), hipHostMallocDefault);
  if (e == hipSuccess) e = hipMemcpyAsync(d->theta, th.data(), th.size() * 4, hipMemcpyHostToDevice, ctx().stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx().stream);
  if (e != hipSuccess) { cai_decoder_destroy(d); return hip_fail(e, "cai_decoder_create allocation", __FILE__, __LINE__); }
  d->d_pos = d->d_tokens + 8; d->d_argmax = d->d_tokens + 16; d->d_gen_idx = d->d_tokens + 24;
  const char* ng = getenv("CAIHIP_NO_GRAPH");
  d->use_graph = !(ng && ng[0] == '1');
  *out = d;
  return CAI_OK;
}

extern "C" int cai_decoder_destroy(cai_decoder_t d)
{
  CAI_ENTER();
  if (!d) return CAI_OK;
  if (ctx().ready) (void)hipStreamSynchronize(ctx().stream);
  invalidate_graphs(d);
  kv_free(&d->kv);
  float* fs[] = {d->wpart, d->ssq, d->theta, d->x, d->qkv, d->att, d->gu, d->mid, d->logits, d->router_logits, d->router_probs, d->moe_gate, d->moe_part, d->final_norm};
  for (float* p : fs) if (p) (void)hipFree(p);
  for (auto& L : d->layers) for (float* p : L.v) if (p) (void)hipFree(p);
  { float* pf[] = {d->px, d->pqkv, d->patt, d->pgu, d->pmid, d->ppart}; for (float* q : pf) if (q) (void)hipFree(q); }
  if (d->ptokpos) (void)hipFree(d->ptokpos);
  free_moe_prompt(d);
  if (d->moe_expert) (void)hipFree(d->moe_expert);
  if (d->am_v) (void)hipFree(d->am_v);
  if (d->am_i) (void)hipFree(d->am_i);
  if (d->d_tokens) (void)hipFree(d->d_tokens);
  if (d->d_gen) (void)hipFree(d->d_gen);
  if (d->h_io) (void)hipHostFree(d->h_io);
  for (cai_qw_s* w : d->owned) (void)cai_qw_destroy(w);
  delete d;
  return CAI_OK;
}

namespace cai {
void decoder_adopt_weight(cai_decoder_s* d, cai_qw_s* w) { d->owned.push_back(w); }
}  // namespace cai

extern "C" int cai_decoder_set_weight(cai_decoder_t d, int layer, int slot, cai_qw_t w)
{
  CAI_ENTER();
  CAI_REQUIRE(d && w, "cai_decoder_set_weight: null argument");
  const cai_decoder_config& c = d->cfg;
  const int qw = d->qw(), kw = d->kw();
  int64_t rows = -1, cols = -1;
  const int64_t E = c.n_experts > 0 ? c.n_experts : 1;
  switch (slot) {
    case CAI_W_EMBED: case CAI_W_HEAD: rows = c.vocab; cols = c.d_model; break;
    case CAI_W_Q: rows = qw; cols = c.d_model; break;
    case CAI_W_K: case CAI_W_V: rows = kw; cols = c.d_model; break;
    case CAI_W_O: rows = c.d_model; cols = qw; break;
    case CAI_W_GATEUP: rows = E * 2 * c.ffn; cols = c.d_model; break;
    case CAI_W_DOWN: rows = E * c.d_model; cols = c.ffn; break;
    case CAI_W_ROUTER: rows = c.n_experts; cols = c.d_model; break;
    default: return set_error(CAI_ERR_INVALID, "cai_decoder_set_weight: unknown slot %d", slot);
  }
  CAI_REQUIRE(w->rows == rows && w->cols == cols, "cai_decoder_set_weight: slot %d expects %lld x %lld, got %lld x %lld", slot,
              (long long)rows, (long long)cols, (long long)w->rows, (long long)w->cols);
  if (slot == CAI_W_EMBED) d->embed = w;
  else if (slot == CAI_W_HEAD) d->head = w;
  else {
    CAI_REQUIRE(layer >= 0 && layer < c.n_layers, "cai_decoder_set_weight: layer %d of %d", layer, c.n_layers);
    d->layers[layer].w[slot] = w;
  }
  invalidate_graphs(d);
  return CAI_OK;
}

extern "C" int cai_decoder_set_vector(cai_decoder_t d, int layer, int slot, const float* v, int n)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && v, "cai_decoder_set_vector: null argument");
  const cai_decoder_config& c = d->cfg;
  int want = c.d_model;
  if (slot == CAI_V_Q_NORM) want = d->qw(); else if (slot == CAI_V_K_NORM) want = d->kw();
  CAI_REQUIRE(slot >= 0 && slot <= 4, "cai_decoder_set_vector: unknown slot %d", slot);
  CAI_REQUIRE(n == want, "cai_decoder_set_vector: slot %d expects %d values, got %d", slot, want, n);
  float** dst;
  if (slot == CAI_V_FINAL_NORM) dst = &d->final_norm;
  else {
    CAI_REQUIRE(layer >= 0 && layer < c.n_layers, "cai_decoder_set_vector: layer %d of %d", layer, c.n_layers);
    dst = &d->layers[layer].v[slot];
  }
  if (!*dst) CAI_HIP(hipMalloc((void**)dst, (size_t)n * 4));
  CAI_HIP(hipMemcpyAsync(*dst, v, (size_t)n * 4, hipMemcpyHostToDevice, ctx().stream));
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  invalidate_graphs(d);
  return CAI_OK;
}

extern "C" int cai_decoder_step(cai_decoder_t d, const int32_t* tokens, const int32_t* pos, int n_b, float* logits, int32_t* argmax)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && tokens && pos, "cai_decoder_step: null argument");
  const cai_decoder_config& c = d->cfg;
  CAI_REQUIRE(n_b >= 1 && n_b <= c.max_batch, "cai_decoder_step: n_b %d outside 1..%d", n_b, c.max_batch);
  int rc = check_ready(d); if (rc) return rc;
  for (int b = 0; b < n_b; b++) {
    CAI_REQUIRE(tokens[b] >= 0 && tokens[b] < c.vocab, "cai_decoder_step: token %d outside vocab %d", tokens[b], c.vocab);
    if (pos[b] != d->kv.len_at(b, 0)) return set_error(CAI_ERR_STATE, "cai_decoder_step: sequence %d is at position %d, got %d", b, d->kv.len_at(b, 0), pos[b]);
    if (pos[b] >= c.max_ctx && d->kv.evict_cap == 0) return set_error(CAI_ERR_STATE, "cai_decoder_step: sequence %d reached max_ctx %d", b, c.max_ctx);
  }
  Context& cx = ctx();
  for (int b = 0; b < n_b; b++) { d->h_io[b] = tokens[b]; d->h_io[8 + b] = pos[b]; }
  CAI_HIP(hipMemcpyAsync(d->d_tokens, d->h_io, 16 * sizeof(int32_t), hipMemcpyHostToDevice, cx.stream));
  int rows_needed = 0;
  for (int b = 0; b < n_b; b++) rows_needed = std::max(rows_needed, pos[b] + 1);
  if ((rc = run_step(d, n_b, rows_needed))) return rc;
  if (logits) CAI_HIP(hipMemcpyAsync(logits, d->logits, (size_t)n_b * c.vocab * 4, hipMemcpyDeviceToHost, cx.stream));
  CAI_HIP(hipMemcpyAsync(d->h_io + 16, d->d_argmax, 8 * sizeof(int32_t), hipMemcpyDeviceToHost, cx.stream));
  CAI_HIP(hipStreamSynchronize(cx.stream));
  for (int b = 0; b < n_b; b++) {
    for (int l = 0; l < c.n_layers; l++) d->kv.len_at(b, l) = pos[b] + 1;
    if (argmax) argmax[b] = d->h_io[16 + b];
  }
  return CAI_OK;
}

// Width-n window step of ONE sequence (StepForward on a width-K twin, neural/neuraldecode.pas:1151-1183 and 5696-5712; the verify
// pass of speculative decoding, examples/SpeculativeDecoding/SpeculativeDecoding.lpr:646-663): tokens[r] is fed at position
// pos0 + r, appended to the cache, and attends to everything before it; row r of the result is the model's output at position
// pos0 + r.  The cache then holds pos0 + n rows: the caller keeps the prefix it commits with cai_decoder_truncate.
extern "C" int cai_decoder_step_window(cai_decoder_t d, int seq, const int32_t* tokens, int n, int pos0, float* logits, int32_t* argmax)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && tokens, "cai_decoder_step_window: null argument");
  const cai_decoder_config& c = d->cfg;
  CAI_REQUIRE(n >= 1 && n <= 8, "cai_decoder_step_window: width %d outside 1..8", n);
  CAI_REQUIRE(seq >= 0 && seq < c.max_batch, "cai_decoder_step_window: sequence %d of %d", seq, c.max_batch);
  int rc = check_ready(d); if (rc) return rc;
  if (pos0 != d->kv.len_at(seq, 0)) return set_error(CAI_ERR_STATE, "cai_decoder_step_window: sequence %d is at position %d, got %d", seq, d->kv.len_at(seq, 0), pos0);
  if (d->kv.evict_cap > 0 && n > 1) return set_error(CAI_ERR_UNSUPPORTED, "cai_decoder_step_window: a session with eviction rolls its cache and cannot take back a window; step one token at a time");
  if (pos0 + n > c.max_ctx && d->kv.evict_cap == 0) return set_error(CAI_ERR_STATE, "cai_decoder_step_window: %d tokens from %d exceed max_ctx %d", n, pos0, c.max_ctx);
  for (int i = 0; i < n; i++) CAI_REQUIRE(tokens[i] >= 0 && tokens[i] < c.vocab, "cai_decoder_step_window: token %d outside vocab %d", tokens[i], c.vocab);
  Context& cx = ctx();
  if (n > 1 && (rc = ensure_wpart(d))) return rc;
  CAI_HIP(hipStreamSynchronize(cx.stream));   // h_io is reused
  for (int i = 0; i < n; i++) { d->h_io[i] = tokens[i]; d->h_io[8 + i] = pos0 + i; }
  CAI_HIP(hipMemcpyAsync(d->d_tokens, d->h_io, 16 * sizeof(int32_t), hipMemcpyHostToDevice, cx.stream));
  if ((rc = run_step(d, n, pos0 + n, n > 1, seq))) return rc;
  if (logits) CAI_HIP(hipMemcpyAsync(logits, d->logits, (size_t)n * c.vocab * 4, hipMemcpyDeviceToHost, cx.stream));
  CAI_HIP(hipMemcpyAsync(d->h_io + 16, d->d_argmax, 8 * sizeof(int32_t), hipMemcpyDeviceToHost, cx.stream));
  CAI_HIP(hipStreamSynchronize(cx.stream));
  for (int l = 0; l < c.n_layers; l++) d->kv.len_at(seq, l) = pos0 + n;
  if (argmax) for (int i = 0; i < n; i++) argmax[i] = d->h_io[16 + i];
  return CAI_OK;
}

extern "C" int cai_prompt_lookup_draft(const int32_t* context, int n_ctx, int match_len, int num_draft, int32_t* draft_out, int* n_draft_out)
{
  CAI_ENTER();
  CAI_REQUIRE(context && draft_out && n_draft_out && n_ctx >= 0, "cai_prompt_lookup_draft: bad argument");
  *n_draft_out = lookup_draft(context, n_ctx, match_len, num_draft, draft_out);
  return CAI_OK;
}

// Greedy continuation with prompt-lookup drafts (DecodePromptLookup, neural/neuraldecode.pas:7767-7866, on the cached session):
// every pass feeds the last committed token plus the draft as ONE window, keeps the drafted tokens the model itself would
// have produced, and rolls the cache back over the rest.  Every emitted token is the arg-max of a row whose inputs are
// committed tokens, so the output is that of plain greedy decoding; only the number of passes differs.
extern "C" int cai_decoder_generate_lookup(cai_decoder_t d, const int32_t* context, int n_ctx, int match_len, int num_draft,
                                           int n_tokens, int32_t* tokens_out, int32_t* passes_out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && context && tokens_out && n_ctx >= 1 && n_tokens >= 1, "cai_decoder_generate_lookup: bad argument");
  const cai_decoder_config& c = d->cfg;
  if (d->kv.len_at(0, 0) != n_ctx - 1)
    return set_error(CAI_ERR_STATE, "cai_decoder_generate_lookup: the cache of sequence 0 holds %d tokens, the context's first %d are expected (its last token is fed here)", d->kv.len_at(0, 0), n_ctx - 1);
  if (d->kv.evict_cap == 0 ? n_ctx - 1 + n_tokens > c.max_ctx : n_tokens > c.max_ctx)   // (a session with eviction runs past max_ctx, like cai_decoder_generate)
    return set_error(CAI_ERR_STATE, "cai_decoder_generate_lookup: %d tokens from %d exceed max_ctx %d", n_tokens, n_ctx - 1, c.max_ctx);
  if (match_len < 1) match_len = 1;                       // (the reference clamps both the same way)
  if (num_draft < 1) num_draft = 1;
  const bool can_draft = d->kv.evict_cap == 0;            // a rolling cache cannot take a window back
  std::vector<int32_t> all(context, context + n_ctx);
  all.reserve((size_t)n_ctx + n_tokens);
  int emitted = 0, passes = 0;
  while (emitted < n_tokens) {
    const int pos = (int)all.size() - 1;
    int32_t win[8], am[8];
    win[0] = all.back();
    const int room = can_draft ? std::min(std::min(num_draft, 7), std::min(n_tokens - emitted - 1, c.max_ctx - pos - 1)) : 0;
    const int nd = room > 0 ? lookup_draft(all.data(), (int)all.size(), match_len, room, win + 1) : 0;
    const int rc = cai_decoder_step_window(d, 0, win, 1 + nd, pos, nullptr, am);
    if (rc) return rc;
    passes++;
    int acc = 0;
    all.push_back(am[0]); tokens_out[emitted++] = am[0];
    while (acc < nd && emitted < n_tokens && win[1 + acc] == am[acc]) { acc++; all.push_back(am[acc]); tokens_out[emitted++] = am[acc]; }
    for (int l = 0; l < c.n_layers; l++) d->kv.len_at(0, l) = pos + 1 + acc;   // rows of rejected drafts are dropped
  }
  if (passes_out) *passes_out = passes;
  return CAI_OK;
}

extern "C" int cai_decoder_generate(cai_decoder_t d, int32_t first_token, int pos, int n_tokens, int32_t* tokens_out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && tokens_out && n_tokens >= 1, "cai_decoder_generate: bad argument");
  const cai_decoder_config& c = d->cfg;
  int rc = check_ready(d); if (rc) return rc;
  CAI_REQUIRE(first_token >= 0 && first_token < c.vocab, "cai_decoder_generate: token %d outside vocab %d", first_token, c.vocab);
  if (pos != d->kv.len_at(0, 0)) return set_error(CAI_ERR_STATE, "cai_decoder_generate: sequence 0 is at position %d, got %d", d->kv.len_at(0, 0), pos);
  if (d->kv.evict_cap == 0 ? pos + n_tokens > c.max_ctx : n_tokens > c.max_ctx)
    return set_error(CAI_ERR_STATE, "cai_decoder_generate: %d tokens from %d exceed max_ctx %d", n_tokens, pos, c.max_ctx);
  Context& cx = ctx();
  d->h_io[0] = first_token; d->h_io[8] = pos; d->h_io[24] = 0;
  CAI_HIP(hipMemcpyAsync(d->d_tokens, d->h_io, 16 * sizeof(int32_t), hipMemcpyHostToDevice, cx.stream));
  CAI_HIP(hipMemcpyAsync(d->d_gen_idx, d->h_io + 24, sizeof(int32_t), hipMemcpyHostToDevice, cx.stream));
  for (int i = 0; i < n_tokens;) {
    const int steps = n_tokens - i >= GEN_UNROLL ? GEN_UNROLL : 1;
    if ((rc = run_gen_steps(d, steps, pos + i + steps))) return rc;
    i += steps;
  }
  CAI_HIP(hipMemcpyAsync(tokens_out, d->d_gen, (size_t)n_tokens * sizeof(int32_t), hipMemcpyDeviceToHost, cx.stream));
  CAI_HIP(hipStreamSynchronize(cx.stream));
  for (int l = 0; l < c.n_layers; l++) d->kv.len_at(0, l) = pos + n_tokens;
  return CAI_OK;
}

// Per-class timing of the batch-1 step: what the captured step gains when one class of launches is left out (see below).
extern "C" int cai_decoder_profile(cai_decoder_t d, int32_t token, int reps, float* us_per_step_out, int n_classes)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && us_per_step_out && reps >= 1 && n_classes >= 1 && n_classes <= 8, "cai_decoder_profile: bad argument");
  const cai_decoder_config& c = d->cfg;
  int rc = check_ready(d); if (rc) return rc;
  CAI_REQUIRE(token >= 0 && token < c.vocab, "cai_decoder_profile: token %d outside vocab %d", token, c.vocab);
  const int pos = d->kv.len_at(0, 0);
  if (pos >= c.max_ctx && d->kv.evict_cap == 0) return set_error(CAI_ERR_STATE, "cai_decoder_profile: sequence 0 reached max_ctx %d", c.max_ctx);
  Context& cx = ctx();
  d->h_io[0] = token; d->h_io[8] = pos;
  CAI_HIP(hipMemcpyAsync(d->d_tokens, d->h_io, 16 * sizeof(int32_t), hipMemcpyHostToDevice, cx.stream));
  d->kv.geo_rows = kv_bucket_rows(&d->kv, pos + 1);
  if ((rc = enqueue_step(d, 1, 0))) return rc;      // a whole step first: every buffer a class reads holds this step's values
  // `reps` steps restricted to `classes`, as ONE captured graph replayed between two events (the way the decode step itself runs;
  // launches enqueued one by one are paced by the host thread, 17.6 to 20.1 us for the same 17.4 us kernel from machine to machine)
  auto time_steps = [&](unsigned classes, float* us_per_step) -> int {
    int rcl = CAI_OK;
    hipGraphExec_t ge = nullptr;
    if (d->use_graph) {
      hipGraph_t g = nullptr;
      CAI_HIP(hipStreamBeginCapture(cx.stream, hipStreamCaptureModeThreadLocal));
      for (int r = 0; r < reps && !rcl; r++) rcl = enqueue_step(d, 1, 0, classes);
      const hipError_t e = hipStreamEndCapture(cx.stream, &g);
      if (rcl) { if (g) (void)hipGraphDestroy(g); return rcl; }
      if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture", __FILE__, __LINE__);
      const hipError_t e2 = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
      (void)hipGraphDestroy(g);
      if (e2 != hipSuccess) return hip_fail(e2, "hipGraphInstantiate", __FILE__, __LINE__);
      const hipError_t e3 = hipGraphLaunch(ge, cx.stream);          // the first launch also uploads the graph: not timed
      if (e3 != hipSuccess) { (void)hipGraphExecDestroy(ge); return hip_fail(e3, "hipGraphLaunch", __FILE__, __LINE__); }
    } else if ((rcl = enqueue_step(d, 1, 0, classes))) return rcl;  // warm
    float t[3] = {0.0f, 0.0f, 0.0f};                               // three timed replays, the median counts
    hipError_t e = hipSuccess;
    for (int i = 0; i < 3 && e == hipSuccess && !rcl; i++) {
      e = hipEventRecord(cx.ev0, cx.stream);
      if (ge) { if (e == hipSuccess) e = hipGraphLaunch(ge, cx.stream); }
      else for (int r = 0; r < reps && !rcl; r++) rcl = enqueue_step(d, 1, 0, classes);
      if (e == hipSuccess) e = hipEventRecord(cx.ev1, cx.stream);
      if (e == hipSuccess) e = hipEventSynchronize(cx.ev1);
      if (e == hipSuccess) e = hipEventElapsedTime(&t[i], cx.ev0, cx.ev1);
    }
    if (ge) (void)hipGraphExecDestroy(ge);
    if (rcl) return rcl;
    if (e != hipSuccess) return hip_fail(e, "cai_decoder_profile timing", __FILE__, __LINE__);
    const float ms = std::max(std::min(t[0], t[1]), std::min(std::max(t[0], t[1]), t[2]));
    *us_per_step = ms * 1e3f / (float)reps;
    return CAI_OK;
  };
  // A class costs what the step gains when its launches are left out: both sides are whole steps replayed as graphs, so the
  // figure is the kernel in its place in the chain (its dependent-launch gap included) and the classes add up to the step.
  // Class launches timed back to back by themselves came out at 17.7 or at 20 us per gate|up launch from one process to the next
  // while the step stayed at 1.656 ms throughout.
  float all_us = 0.0f;
  if ((rc = time_steps(~0u, &all_us))) return rc;
  for (int k = 0; k < n_classes; k++) {
    unsigned drop = 1u << k;
    if (c.n_experts > 0 && k == 4) drop = 48u;                       // the expert half is one class (reported under 4)
    if (c.n_experts > 0 && k == 5) { us_per_step_out[k] = 0.0f; continue; }
    float without = 0.0f;
    if ((rc = time_steps(~0u & ~drop, &without))) return rc;
    us_per_step_out[k] = all_us - without;
  }
  if ((rc = enqueue_step(d, 1, 0))) return rc;      // leave the buffers as a whole step leaves them
  CAI_HIP(hipGetLastError());
  return CAI_OK;     // (the session's length is unchanged: the K,V row written at the current position is not counted)
}

// Device-side timeline of one captured batch-1 step (see the header): stamps of the third replay.
extern "C" int cai_decoder_timeline(cai_decoder_t d, int32_t token, uint64_t* stamps_out, int64_t stamps_cap, int32_t* launches_out,
                                    int launches_cap, int* n_launches_out, int64_t* n_stamps_out, float* ticks_per_us_out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && stamps_out && launches_out && n_launches_out && n_stamps_out && ticks_per_us_out && stamps_cap > 0 && launches_cap > 0, "cai_decoder_timeline: bad argument");
  const cai_decoder_config& c = d->cfg;
  int rc = check_ready(d); if (rc) return rc;
  CAI_REQUIRE(token >= 0 && token < c.vocab, "cai_decoder_timeline: token %d outside vocab %d", token, c.vocab);
  const int pos = d->kv.len_at(0, 0);
  if (pos >= c.max_ctx && d->kv.evict_cap == 0) return set_error(CAI_ERR_STATE, "cai_decoder_timeline: sequence 0 reached max_ctx %d", c.max_ctx);
#ifndef CAI_TIMELINE
  return set_error(CAI_ERR_UNSUPPORTED, "cai_decoder_timeline: this build carries no stamps (build libcaihip_timeline.so: make -C neural-api_amd/csrc timeline)");
#endif
  Context& cx = ctx();
  Context::Timeline& tl = cx.tl;
  if ((size_t)stamps_cap > tl.cap) {
    CAI_HIP(hipStreamSynchronize(cx.stream));
    if (tl.buf) { (void)hipFree(tl.buf); tl.buf = nullptr; tl.cap = 0; }
    CAI_HIP(hipMalloc((void**)&tl.buf, (size_t)stamps_cap * sizeof(unsigned long long)));
    tl.cap = (size_t)stamps_cap;
  }
  // (CAIHIP_TL_BATCH = b: the step of sequences 0 .. b - 1, each at its own position, all fed `token`)
  const char* tb = getenv("CAIHIP_TL_BATCH");
  const int n_b = tb ? std::max(1, std::min(atoi(tb), std::min(c.max_batch, 8))) : 1;
  int rows_needed = pos + 1;
  for (int b = 0; b < n_b; b++) { d->h_io[b] = token; d->h_io[8 + b] = d->kv.len_at(b, 0); rows_needed = std::max(rows_needed, d->kv.len_at(b, 0) + 1); }
  CAI_HIP(hipMemcpyAsync(d->d_tokens, d->h_io, 16 * sizeof(int32_t), hipMemcpyHostToDevice, cx.stream));
  d->kv.geo_rows = kv_bucket_rows(&d->kv, rows_needed);
  tl.used = 0; tl.launches.clear(); tl.armed = true;
  hipGraph_t g = nullptr; hipGraphExec_t ge = nullptr;
  hipError_t e = hipStreamBeginCapture(cx.stream, hipStreamCaptureModeThreadLocal);
  if (e != hipSuccess) { tl.armed = false; return hip_fail(e, "hipStreamBeginCapture", __FILE__, __LINE__); }
  rc = enqueue_step(d, n_b, 0);
  tl.armed = false;
  e = hipStreamEndCapture(cx.stream, &g);
  if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
  if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture", __FILE__, __LINE__);
  e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (e != hipSuccess) return hip_fail(e, "hipGraphInstantiate", __FILE__, __LINE__);
  for (int i = 0; i < 3 && e == hipSuccess; i++) {
    if (i == 2) e = hipMemsetAsync(tl.buf, 0, tl.used * sizeof(unsigned long long), cx.stream);
    if (e == hipSuccess) e = hipGraphLaunch(ge, cx.stream);
  }
  if (e == hipSuccess) e = hipMemcpyAsync(stamps_out, tl.buf, tl.used * sizeof(unsigned long long), hipMemcpyDeviceToHost, cx.stream);
  if (e == hipSuccess) e = hipStreamSynchronize(cx.stream);
  (void)hipGraphExecDestroy(ge);
  if (e != hipSuccess) return hip_fail(e, "cai_decoder_timeline replay", __FILE__, __LINE__);
  const int n = std::min((int)(tl.launches.size() / 3), launches_cap);
  for (int i = 0; i < 3 * n; i++) launches_out[i] = tl.launches[i];
  *n_launches_out = n; *n_stamps_out = (int64_t)tl.used;
  int khz = 100000;
  (void)hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, cx.device);
  *ticks_per_us_out = (float)khz * 1e-3f;
  return CAI_OK;     // (the session's length is unchanged: the K,V row written at the current position is not counted)
}

extern "C" int cai_decoder_prefill(cai_decoder_t d, int seq, const int32_t* tokens, int n, int pos0, float* last_logits, int32_t* argmax)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && tokens && n >= 1, "cai_decoder_prefill: bad argument");
  const cai_decoder_config& c = d->cfg;
  CAI_REQUIRE(seq >= 0 && seq < c.max_batch, "cai_decoder_prefill: sequence %d of %d", seq, c.max_batch);
  int rc = check_ready(d); if (rc) return rc;
  if (pos0 != d->kv.len_at(seq, 0)) return set_error(CAI_ERR_STATE, "cai_decoder_prefill: sequence %d is at position %d, got %d", seq, d->kv.len_at(seq, 0), pos0);
  if (pos0 + n > c.max_ctx && d->kv.evict_cap == 0) return set_error(CAI_ERR_STATE, "cai_decoder_prefill: %d tokens from %d exceed max_ctx %d", n, pos0, c.max_ctx);
  for (int i = 0; i < n; i++) CAI_REQUIRE(tokens[i] >= 0 && tokens[i] < c.vocab, "cai_decoder_prefill: token %d outside vocab %d", tokens[i], c.vocab);
  Context& cx = ctx();
  const char* tok_env = getenv("CAIHIP_PREFILL_TOKENWISE");
  // (a prompt that runs past the eviction cap overwrites ring rows its own earlier tokens still need: token by token then)
  const bool tokenwise = n == 1 || (tok_env && tok_env[0] == '1') || (d->kv.evict_cap > 0 && pos0 + n > d->kv.evict_cap);
  if (tokenwise) {
    // Token-at-a-time ingestion, the reference's own prefill (neural/neuralchatengine.pas:1466-1470).
    for (int i = 0; i < n; i++) {
      CAI_HIP(hipStreamSynchronize(cx.stream));   // h_io is reused
      d->h_io[0] = tokens[i]; d->h_io[8] = pos0 + i;
      CAI_HIP(hipMemcpyAsync(d->d_tokens, d->h_io, 16 * sizeof(int32_t), hipMemcpyHostToDevice, cx.stream));
      if ((rc = run_step(d, 1, pos0 + i + 1, false, seq))) return rc;
    }
  } else {
    const int chunk = 512;
    if ((rc = ensure_prefill_buffers(d, std::min(n, chunk)))) return rc;
    std::vector<int32_t> tp((size_t)2 * d->pf_cap);
    for (int t0 = 0; t0 < n; t0 += chunk) {
      const int m = std::min(chunk, n - t0);
      for (int i = 0; i < m; i++) { tp[i] = tokens[t0 + i]; tp[d->pf_cap + i] = pos0 + t0 + i; }
      CAI_HIP(hipMemcpyAsync(d->ptokpos, tp.data(), tp.size() * sizeof(int32_t), hipMemcpyHostToDevice, cx.stream));
      CAI_HIP(hipStreamSynchronize(cx.stream));
      d->kv.geo_rows = kv_bucket_rows(&d->kv, pos0 + t0 + m);
      if ((rc = ensure_ppart(d, pos0 + t0 + m, m))) return rc;
      if ((rc = enqueue_prefill_chunk(d, seq, m))) return rc;
      CAI_HIP(hipGetLastError());
      if (t0 + chunk >= n) {
        // logits of the last prompt token only: final RMSNorm + vocabulary projection + arg-max on its row
        cai_qw_s* hw = d->head ? d->head : d->embed;
        MultiGemv hm{}; hm.n = 1; hm.w[0] = hw; hm.rows[0] = c.vocab;
        if ((rc = launch_gemv_multi(hm, d->px + (int64_t)(m - 1) * c.d_model, 1, d->logits, c.vocab, CAI_ACT_NONE, nullptr, d->final_norm, c.eps, 0))) return rc;
        launch_argmax(d->logits, c.vocab, 1, d->d_argmax, d->am_v, d->am_i);
        // the last token's residual stream goes where a step leaves it (cai_decoder_hidden_state reads row 0)
        CAI_HIP(hipMemcpyAsync(d->x, d->px + (int64_t)(m - 1) * c.d_model, (size_t)c.d_model * 4, hipMemcpyDeviceToDevice, cx.stream));
      }
    }
  }
  if (last_logits) CAI_HIP(hipMemcpyAsync(last_logits, d->logits, (size_t)c.vocab * 4, hipMemcpyDeviceToHost, cx.stream));
  CAI_HIP(hipMemcpyAsync(d->h_io + 16, d->d_argmax, 8 * sizeof(int32_t), hipMemcpyDeviceToHost, cx.stream));
  CAI_HIP(hipStreamSynchronize(cx.stream));
  for (int l = 0; l < c.n_layers; l++) d->kv.len_at(seq, l) = pos0 + n;
  if (argmax) *argmax = d->h_io[16];
  return CAI_OK;
}

// HiddenState (neural/neuraldecode.pas:1314-1321, 5850-5857): the input of the vocabulary projection - the final RMSNorm of the
// residual stream - for row `row` of the last step or window (row 0 after cai_decoder_prefill / cai_decoder_generate: the last
// token fed).  The decode step fuses that norm into the projection, so it is recomputed here from the stream the step left.
extern "C" int cai_decoder_hidden_state(cai_decoder_t d, int row, float* hidden_out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && hidden_out, "cai_decoder_hidden_state: null argument");
  CAI_REQUIRE(row >= 0 && row < 8, "cai_decoder_hidden_state: row %d outside 0..7", row);
  if (!d->final_norm) return set_error(CAI_ERR_STATE, "cai_decoder_hidden_state: final norm gain not set");
  Context& cx = ctx();
  const int dm = d->cfg.d_model;
  int rc = ensure_stage(&cx.stage_out, &cx.stage_out_cap, (size_t)dm * 4); if (rc) return rc;
  if ((rc = launch_rmsnorm(d->x + (int64_t)row * dm, d->final_norm, dm, 1, d->cfg.eps, (float*)cx.stage_out))) return rc;
  CAI_HIP(hipMemcpyAsync(hidden_out, cx.stage_out, (size_t)dm * 4, hipMemcpyDeviceToHost, cx.stream));
  CAI_HIP(hipStreamSynchronize(cx.stream));
  return CAI_OK;
}

// The sampled (non-greedy) branch of the decode loop without the logits read-back (neural/neuralchatengine.pas:1495-1501).
extern "C" int cai_decoder_candidates(cai_decoder_t d, int row, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                                      float repetition, float frequency, float presence, float temperature, int m,
                                      int32_t* tokens_out, float* probs_out, int* count_out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && tokens_out && probs_out, "cai_decoder_candidates: null argument");
  CAI_REQUIRE(row >= 0 && row < 8, "cai_decoder_candidates: row %d outside 0..7", row);   // a row of the last step (sequence) or window (position)
  CAI_REQUIRE(m >= 1 && m <= 1024, "cai_decoder_candidates: %d candidates (1..1024)", m);
  return run_candidates(d->logits + (int64_t)row * d->cfg.vocab, d->cfg.vocab, hist_ids, hist_counts, n_hist,
                        repetition, frequency, presence, temperature, m, tokens_out, probs_out, count_out);
}

extern "C" int cai_decoder_reset(cai_decoder_t d, int seq)
{
  CAI_ENTER();
  CAI_REQUIRE(d, "cai_decoder_reset: null decoder");
  CAI_REQUIRE(seq >= 0 && seq < d->cfg.max_batch, "cai_decoder_reset: sequence %d of %d", seq, d->cfg.max_batch);
  for (int l = 0; l < d->cfg.n_layers; l++) d->kv.len_at(seq, l) = 0;
  return CAI_OK;
}

extern "C" int cai_decoder_truncate(cai_decoder_t d, int seq, int n)
{
  CAI_ENTER();
  CAI_REQUIRE(d, "cai_decoder_truncate: null decoder");
  CAI_REQUIRE(seq >= 0 && seq < d->cfg.max_batch && n >= 0, "cai_decoder_truncate: bad argument");
  const int have = d->kv.len_at(seq, 0);
  if (have > n && d->kv.evict_cap > 0 && have > d->kv.evict_cap)
    return set_error(CAI_ERR_STATE, "cai_decoder_truncate: %d tokens streamed under eviction, the rows before %d are gone", have, have - (d->kv.evict_cap - d->kv.evict_sinks));
  for (int l = 0; l < d->cfg.n_layers; l++) if (d->kv.len_at(seq, l) > n) d->kv.len_at(seq, l) = n;
  return CAI_OK;
}

extern "C" int cai_decoder_set_eviction(cai_decoder_t d, int sink_tokens, int recent_window)
{
  CAI_ENTER();
  CAI_REQUIRE(d, "cai_decoder_set_eviction: null decoder");
  const int rc = kv_set_eviction(&d->kv, sink_tokens, recent_window);
  if (rc) return rc;
  (void)hipStreamSynchronize(ctx().stream);
  invalidate_graphs(d);       // captured steps carry the policy in their kernel arguments
  return CAI_OK;
}

// EnableInt8KVCache / DisableInt8KVCache (neural/neuraldecode.pas:1277-1290): the storage mode of an empty session.
extern "C" int cai_decoder_set_kv_dtype(cai_decoder_t d, int kv_dtype)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d, "cai_decoder_set_kv_dtype: null decoder");
  CAI_REQUIRE(kv_dtype == CAI_KV_F32 || kv_dtype == CAI_KV_F16 || kv_dtype == CAI_KV_I8, "cai_decoder_set_kv_dtype: type %d", kv_dtype);
  for (int n : d->kv.len)
    if (n > 0) return set_error(CAI_ERR_STATE, "cai_decoder_set_kv_dtype: the cache holds %d tokens; the storage mode only changes on an empty session", n);
  if (kv_dtype == d->kv.dtype) return CAI_OK;
  (void)hipStreamSynchronize(ctx().stream);
  invalidate_graphs(d);
  const cai_decoder_config& c = d->cfg;
  const int sinks = d->kv.evict_sinks, cap = d->kv.evict_cap;
  const int old = d->kv.dtype;
  kv_free(&d->kv);
  int rc = kv_alloc(&d->kv, c.max_batch, c.n_layers, c.n_kv_heads, c.head_dim, c.max_ctx, kv_dtype);
  if (rc) {
    // back to the type that fitted before; if even that fails the session has no cache and every later call says so
    kv_free(&d->kv);
    if (kv_alloc(&d->kv, c.max_batch, c.n_layers, c.n_kv_heads, c.head_dim, c.max_ctx, old)) { kv_free(&d->kv); d->cache_lost = true; }
    else { d->kv.evict_sinks = sinks; d->kv.evict_cap = cap; }
    return rc;
  }
  d->kv.evict_sinks = sinks; d->kv.evict_cap = cap;
  d->cfg.kv_dtype = kv_dtype;
  // the number of cache slices depends on the storage type, and the prompt and window scratch were sized for the old one
  d->pf_cap = 0; d->wpart_elems = 0;
  return CAI_OK;
}

// Long-context frequency rules of TNNetRotaryEmbedding as the importers configure them (neural/neuralpretrained.pas:633-668):
// the table is rebuilt on the host in double; captured graphs read it through the same pointer and stay valid.
static int set_thetas(cai_decoder_s* d, const std::vector<float>& th, const char* who)
{
  for (int n : d->kv.len)
    if (n > 0) return set_error(CAI_ERR_STATE, "%s: the cache holds %d tokens rotated with the old frequencies; set the rule on an empty session", who, n);
  CAI_HIP(hipMemcpyAsync(d->theta, th.data(), th.size() * 4, hipMemcpyHostToDevice, ctx().stream));
  CAI_HIP(hipStreamSynchronize(ctx().stream));   // th is the caller's stack
  return CAI_OK;
}

extern "C" int cai_decoder_set_rope_scaling(cai_decoder_t d, int mode, float factor, int original_ctx, float low_freq_factor, float high_freq_factor)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d, "cai_decoder_set_rope_scaling: null decoder");
  std::vector<float> th;
  int rc = rope_thetas_scaled(d->cfg.rope_theta, d->cfg.head_dim, mode, factor, original_ctx, low_freq_factor, high_freq_factor, th);
  if (rc) return rc;
  if ((rc = set_thetas(d, th, "cai_decoder_set_rope_scaling"))) return rc;
  const float s = mode == CAI_ROPE_YARN ? (float)(0.1 * log((double)factor) + 1.0) : 1.0f;
  return cai_decoder_set_rope_out_scale(d, s);
}

extern "C" int cai_decoder_set_rope_out_scale(cai_decoder_t d, float scale)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d, "cai_decoder_set_rope_out_scale: null decoder");
  CAI_REQUIRE(scale > 0.0f && scale < 3.0e38f, "cai_decoder_set_rope_out_scale: scale %g", (double)scale);
  for (int n : d->kv.len)
    if (n > 0) return set_error(CAI_ERR_STATE, "cai_decoder_set_rope_out_scale: the cache holds %d tokens; set the rule on an empty session", n);
  if (d->kv.score_mul != scale * scale) invalidate_graphs(d);   // the factor is a launch argument of the captured attention kernels
  d->kv.score_mul = scale * scale;
  return CAI_OK;
}

extern "C" int cai_decoder_set_rope_freq_factors(cai_decoder_t d, const float* factors, int n)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && factors, "cai_decoder_set_rope_freq_factors: null argument");
  CAI_REQUIRE(n == d->cfg.head_dim / 2, "cai_decoder_set_rope_freq_factors: %d factors for %d rotary pairs", n, d->cfg.head_dim / 2);
  std::vector<float> th(n);
  for (int k = 0; k < n; k++) {
    CAI_REQUIRE(factors[k] > 0.0f && factors[k] < 3.0e38f, "cai_decoder_set_rope_freq_factors: factor %d is %g", k, (double)factors[k]);
    th[k] = (float)(pow((double)d->cfg.rope_theta, -2.0 * k / d->cfg.head_dim) / (double)factors[k]);
  }
  return set_thetas(d, th, "cai_decoder_set_rope_freq_factors");
}

extern "C" int cai_decoder_cache_rows(cai_decoder_t d, int seq, int layer, int* rows_out)
{
  CAI_ENTER();
  CAI_REQUIRE(d && rows_out, "cai_decoder_cache_rows: null argument");
  CAI_REQUIRE(seq >= 0 && seq < d->cfg.max_batch && layer >= 0 && layer < d->cfg.n_layers, "cai_decoder_cache_rows: sequence %d, layer %d", seq, layer);
  *rows_out = d->kv.live(d->kv.len_at(seq, layer));
  return CAI_OK;
}

extern "C" int cai_decoder_len(cai_decoder_t d, int seq, int* len_out)
{
  CAI_ENTER();
  CAI_REQUIRE(d && len_out, "cai_decoder_len: null argument");
  CAI_REQUIRE(seq >= 0 && seq < d->cfg.max_batch, "cai_decoder_len: sequence %d of %d", seq, d->cfg.max_batch);
  *len_out = d->kv.len_at(seq, 0);
  return CAI_OK;
}

extern "C" int cai_decoder_snapshot(cai_decoder_t d, int seq, cai_kv_snap_t* out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && out, "cai_decoder_snapshot: null argument");
  CAI_REQUIRE(seq >= 0 && seq < d->cfg.max_batch, "cai_decoder_snapshot: sequence %d of %d", seq, d->cfg.max_batch);
  return kv_snapshot(&d->kv, seq, out);
}

extern "C" int cai_decoder_restore(cai_decoder_t d, int seq, cai_kv_snap_t snap)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d && snap, "cai_decoder_restore: null argument");
  CAI_REQUIRE(seq >= 0 && seq < d->cfg.max_batch, "cai_decoder_restore: sequence %d of %d", seq, d->cfg.max_batch);
  return kv_restore(&d->kv, seq, snap);
}

extern "C" int cai_decoder_fork(cai_decoder_t d, int src_seq, int dst_seq)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(d, "cai_decoder_fork: null decoder");
  CAI_REQUIRE(src_seq >= 0 && src_seq < d->cfg.max_batch && dst_seq >= 0 && dst_seq < d->cfg.max_batch,
              "cai_decoder_fork: sequences %d -> %d of %d", src_seq, dst_seq, d->cfg.max_batch);
  return kv_fork(&d->kv, src_seq, dst_seq);
}

extern "C" int cai_decoder_get_config(cai_decoder_t d, cai_decoder_config* out)
{
  CAI_ENTER();
  CAI_REQUIRE(d && out, "cai_decoder_get_config: null argument");
  *out = d->cfg;
  return CAI_OK;
}

extern "C" int cai_decoder_weight_bytes(cai_decoder_t d, int64_t* out)
{
  CAI_ENTER();
  CAI_REQUIRE(d && out, "cai_decoder_weight_bytes: null argument");
  const cai_decoder_config& c = d->cfg;
  int rc = check_ready(d); if (rc) return rc;
  int64_t b = 0;
  const cai_qw_s* hw = d->head ? d->head : d->embed;
  b += hw->algo_bytes + (int64_t)c.d_model * 4;             // head + final norm gain
  b += d->embed->algo_bytes / d->embed->rows;                // one embedding row
  for (auto& L : d->layers) {
    const int dense[] = {CAI_W_Q, CAI_W_K, CAI_W_V, CAI_W_O};
    for (int s : dense) b += L.w[s]->algo_bytes;
    if (c.n_experts > 0) {
      b += L.w[CAI_W_ROUTER]->algo_bytes;
      b += (L.w[CAI_W_GATEUP]->algo_bytes + L.w[CAI_W_DOWN]->algo_bytes) / c.n_experts * c.top_k;
    } else b += L.w[CAI_W_GATEUP]->algo_bytes + L.w[CAI_W_DOWN]->algo_bytes;
    b += 2 * (int64_t)c.d_model * 4;
  }
  *out = b;
  return CAI_OK;
}

