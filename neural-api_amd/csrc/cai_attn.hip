// KV cache + cached grouped-query decode attention for gfx950.
//
// Layer semantics (TNNetFusedSDPA; neural/neural.cl:2354-2499): the token row is [Q | K | V]; K and V are
// appended to a head-major cache (row (g, p) at (g*MaxCtx + p)*Dk), then for each query head h (KV head
// g = h / group) out_h = softmax(q_h . K_g / sqrt(Dk)) V_g over the live rows [jStart, len).
//
// Device formulation: split-K over the key axis.  Work-group (split, kv_head, sequence) streams its slice
// of K and V exactly once with coalesced row loads (32 lanes x 16 B cover one 128-wide row), serves all
// `G` query heads of the group from that one pass, and keeps an online-softmax state (m, l, acc) per
// head; the 8 half-waves of the group meet in LDS, and the last work-group of a (sequence, KV head) to finish merges
// the splits (arrival counter + device-scope fence), so the whole layer step is one launch.  RoPE of q and of
// the new k row and the cache append happen inside the same kernel.
#include "cai_internal.hpp"

namespace cai {

// sum over each half-wave (32 lanes), result in every lane of that half
__device__ __forceinline__ float half_wave_allsum(float v)
{
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x112, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, true));
  const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 31));
  const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
  return (threadIdx.x & 32) ? hi : lo;
}

template <typename T> __device__ __forceinline__ float kv_to_float(T v);
template <> __device__ __forceinline__ float kv_to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float kv_to_float<__half>(__half v) { return __half2float(v); }
template <typename T> __device__ __forceinline__ T kv_from_float(float v);
template <> __device__ __forceinline__ float kv_from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ __half kv_from_float<__half>(float v) { return __float2half_rn(v); }

struct AttnParams {
  float* qkv; int64_t qkv_stride;
  void* kc; void* vc;          // base of [seq][layer][kv_head][max_ctx][hd]
  int64_t seq_elems, layer_off; // element offsets
  int q_heads, kv_heads, hd, max_ctx;
  int window; float softcap; float inv_sqrt;
  const float* theta;          // hd/2 frequencies or null
  const int32_t* pos;          // [seq]
  int split_len, n_splits;
  float* part;                 // [seq][q_head][split][hd+2]
  float* out; int64_t out_stride;
  int seq0;                    // cache sequence index of activation row 0
  int* counters;               // [seq][kv_head] arrival counters of the split merge (zero between launches)
};

// ---- one kernel per token and layer: RoPE (neural/neural.cl:1517-1542) + KV append (2354-2379) +
//      split-K online-softmax decode (2406-2499) + merge of the splits by the last work-group to finish ----
template <int G, int DS, typename KV_T>
__global__ __launch_bounds__(256) void attn_step_kernel(const AttnParams p)
{
  const int split = blockIdx.x, g = blockIdx.y, seq = blockIdx.z;
  const int pos = p.pos[seq];
  const int len = pos + 1;
  const int j_start = (p.window > 0 && len > p.window) ? len - p.window : 0;
  const int s_begin = max(j_start, split * p.split_len), s_end = min(len, (split + 1) * p.split_len);
  if (s_begin >= s_end) return;   // whole work-group leaves together, before any barrier
  const int s_first = j_start / p.split_len, s_last = pos / p.split_len;
  const int n_active = s_last - s_first + 1;

  const int hw = threadIdx.x >> 5, l32 = threadIdx.x & 31;
  const int hd = p.hd, qw = p.q_heads * hd, kw = p.kv_heads * hd;
  const int d0 = l32 * DS;
  const float* row = p.qkv + (int64_t)seq * p.qkv_stride;

  // rotation of this lane's pairs at the token's position (DS even, or DS == 1 with the pair split over 2 lanes)
  float rs[(DS + 1) / 2], rc[(DS + 1) / 2];
#pragma unroll
  for (int i = 0; i < (DS + 1) / 2; i++) {
    rs[i] = 0.0f; rc[i] = 1.0f;
    const int d = d0 + 2 * i;
    if (p.theta && d < hd) { const float angle = (float)pos * p.theta[d >> 1]; sincosf(angle, &rs[i], &rc[i]); }
  }
  // loads DS elements of a head vector and rotates them (pairs (2k, 2k+1))
  auto load_rot = [&](const float* v, float (&o)[DS], bool rotate) {
    if (DS >= 2) {
#pragma unroll
      for (int i = 0; i < DS; i += 2) {
        const int d = d0 + i;
        const float x0 = d < hd ? v[d] : 0.0f, x1 = d + 1 < hd ? v[d + 1] : 0.0f;
        if (rotate) { o[i] = rc[i / 2] * x0 - rs[i / 2] * x1; o[i + (DS > 1 ? 1 : 0)] = rs[i / 2] * x0 + rc[i / 2] * x1; }
        else { o[i] = x0; o[i + (DS > 1 ? 1 : 0)] = x1; }
      }
    } else {
      const int d = d0;
      const float own = d < hd ? v[d] : 0.0f, mate = (d ^ 1) < hd ? v[d ^ 1] : 0.0f;
      if (rotate) o[0] = (d & 1) ? (rs[0] * mate + rc[0] * own) : (rc[0] * own - rs[0] * mate);
      else o[0] = own;
    }
  };

  float q[G][DS], acc[G][DS], m[G], l[G];
#pragma unroll
  for (int h = 0; h < G; h++) {
    m[h] = -1e30f; l[h] = 0.0f;
    load_rot(row + (g * G + h) * hd, q[h], p.theta != nullptr);
#pragma unroll
    for (int i = 0; i < DS; i++) acc[h][i] = 0.0f;
  }
  KV_T* kc = reinterpret_cast<KV_T*>(p.kc) + (seq + p.seq0) * p.seq_elems + p.layer_off + (int64_t)g * p.max_ctx * hd;
  KV_T* vc = reinterpret_cast<KV_T*>(p.vc) + (seq + p.seq0) * p.seq_elems + p.layer_off + (int64_t)g * p.max_ctx * hd;

  // the work-group whose slice holds `pos` appends the new row and keeps it in registers
  float knew[DS], vnew[DS];
  const bool owns_new = pos >= s_begin && pos < s_end;
  if (owns_new) {
    load_rot(row + qw + g * hd, knew, p.theta != nullptr);
    float dummy[DS];
    load_rot(row + qw + kw + g * hd, dummy, false);
#pragma unroll
    for (int i = 0; i < DS; i++) {
      vnew[i] = kv_to_float<KV_T>(kv_from_float<KV_T>(dummy[i]));
      knew[i] = kv_to_float<KV_T>(kv_from_float<KV_T>(knew[i]));
      if (hw == 0 && d0 + i < hd) {
        kc[(int64_t)pos * hd + d0 + i] = kv_from_float<KV_T>(knew[i]);
        vc[(int64_t)pos * hd + d0 + i] = kv_from_float<KV_T>(vnew[i]);
      }
    }
  }

  for (int j = s_begin + hw; j < s_end; j += 8) {
    float kd[DS], vd[DS];
    if (j == pos) {
#pragma unroll
      for (int i = 0; i < DS; i++) { kd[i] = knew[i]; vd[i] = vnew[i]; }
    } else {
#pragma unroll
      for (int i = 0; i < DS; i++) {
        const int d = d0 + i;
        kd[i] = d < hd ? kv_to_float<KV_T>(kc[(int64_t)j * hd + d]) : 0.0f;
        vd[i] = d < hd ? kv_to_float<KV_T>(vc[(int64_t)j * hd + d]) : 0.0f;
      }
    }
#pragma unroll
    for (int h = 0; h < G; h++) {
      float s = 0.0f;
#pragma unroll
      for (int i = 0; i < DS; i++) s = fmaf(q[h][i], kd[i], s);
      s = half_wave_allsum(s) * p.inv_sqrt;
      if (p.softcap > 0.0f) s = p.softcap * tanhf(s / p.softcap);
      const float mn = fmaxf(m[h], s);
      const float corr = expf(m[h] - mn), pj = expf(s - mn);
      l[h] = l[h] * corr + pj;
#pragma unroll
      for (int i = 0; i < DS; i++) acc[h][i] = acc[h][i] * corr + pj * vd[i];
      m[h] = mn;
    }
  }

  // ---- merge the 8 half-waves through LDS ----
  __shared__ float sm[8][G], sl[8][G];
  __shared__ float sacc[8][G][32 * DS];
  __shared__ int s_last_flag;
  if (l32 == 0) {
#pragma unroll
    for (int h = 0; h < G; h++) { sm[hw][h] = m[h]; sl[hw][h] = l[h]; }
  }
#pragma unroll
  for (int h = 0; h < G; h++)
#pragma unroll
    for (int i = 0; i < DS; i++) sacc[hw][h][d0 + i] = acc[h][i];
  __syncthreads();

  for (int o = threadIdx.x; o < G * hd; o += 256) {
    const int h = o / hd, d = o % hd;
    float M = -1e30f;
#pragma unroll
    for (int w = 0; w < 8; w++) M = fmaxf(M, sm[w][h]);
    float L = 0.0f, A = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; w++) {
      const float e = sl[w][h] > 0.0f ? expf(sm[w][h] - M) : 0.0f;
      L = fmaf(sl[w][h], e, L); A = fmaf(sacc[w][h][d], e, A);
    }
    const int qh = g * G + h;
    if (n_active == 1) {
      p.out[(int64_t)seq * p.out_stride + qh * hd + d] = L > 0.0f ? A * (1.0f / L) : 0.0f;
    } else {
      // device-coherent stores: the merging work-group may sit on another XCD (its own L2)
      float* pt = p.part + (((int64_t)seq * p.q_heads + qh) * p.n_splits + split) * (hd + 2);
      __hip_atomic_store(&pt[d], A, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (d == 0) {
        __hip_atomic_store(&pt[hd], M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&pt[hd + 1], L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  if (n_active == 1) return;

  // ---- the last work-group of this (sequence, KV head) to arrive merges the splits ----
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");   // every lane's stores have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    int* cnt = p.counters + seq * p.kv_heads + g;
    const int prev = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    const int last = prev == n_active - 1;
    if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    s_last_flag = last;
  }
  __syncthreads();
  if (!s_last_flag) return;
  // all (M, L) pairs of the group first (independent device-coherent loads), then the accumulators in batches
  __shared__ float mM[G][64], mL[G][64];
  for (int i = threadIdx.x; i < G * n_active; i += 256) {
    const int h = i / n_active, s = s_first + i % n_active;
    const float* pt = p.part + (((int64_t)seq * p.q_heads + g * G + h) * p.n_splits + s) * (hd + 2);
    mM[h][s - s_first] = __hip_atomic_load(&pt[hd], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    mL[h][s - s_first] = __hip_atomic_load(&pt[hd + 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  for (int o = threadIdx.x; o < G * hd; o += 256) {
    const int h = o / hd, d = o % hd, qh = g * G + h;
    const float* pt = p.part + (((int64_t)seq * p.q_heads + qh) * p.n_splits + s_first) * (hd + 2) + d;
    float M = -1e30f;
    for (int s = 0; s < n_active; s++) M = fmaxf(M, mM[h][s]);
    float L = 0.0f, A = 0.0f;
    for (int s0 = 0; s0 < n_active; s0 += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; u++)
        v[u] = s0 + u < n_active ? __hip_atomic_load(&pt[(int64_t)(s0 + u) * (hd + 2)], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
#pragma unroll
      for (int u = 0; u < 8; u++) {
        if (s0 + u < n_active) {
          const float ls = mL[h][s0 + u];
          const float e = ls > 0.0f ? expf(mM[h][s0 + u] - M) : 0.0f;
          L = fmaf(ls, e, L); A = fmaf(v[u], e, A);
        }
      }
    }
    p.out[(int64_t)seq * p.out_stride + qh * hd + d] = L > 0.0f ? A * (1.0f / L) : 0.0f;
  }
}

template <int G, typename KV_T>
static int launch_split_ds(const AttnParams& p, int n_seq, hipStream_t st)
{
  const dim3 grid(p.n_splits, p.kv_heads, n_seq);
  if (p.hd <= 32) hipLaunchKernelGGL((attn_step_kernel<G, 1, KV_T>), grid, dim3(256), 0, st, p);
  else if (p.hd <= 64) hipLaunchKernelGGL((attn_step_kernel<G, 2, KV_T>), grid, dim3(256), 0, st, p);
  else if (p.hd <= 128) hipLaunchKernelGGL((attn_step_kernel<G, 4, KV_T>), grid, dim3(256), 0, st, p);
  else return set_error(CAI_ERR_UNSUPPORTED, "attention: head_dim %d > 128", p.hd);
  return CAI_OK;
}

template <typename KV_T>
static int launch_split_g(const AttnParams& p, int n_seq, hipStream_t st)
{
  switch (p.q_heads / p.kv_heads) {
    case 1: return launch_split_ds<1, KV_T>(p, n_seq, st);
    case 2: return launch_split_ds<2, KV_T>(p, n_seq, st);
    case 3: return launch_split_ds<3, KV_T>(p, n_seq, st);
    case 4: return launch_split_ds<4, KV_T>(p, n_seq, st);
    case 5: return launch_split_ds<5, KV_T>(p, n_seq, st);
    case 6: return launch_split_ds<6, KV_T>(p, n_seq, st);
    case 7: return launch_split_ds<7, KV_T>(p, n_seq, st);
    case 8: return launch_split_ds<8, KV_T>(p, n_seq, st);
  }
  return set_error(CAI_ERR_UNSUPPORTED, "attention: %d query heads per KV head (supported 1..8)", p.q_heads / p.kv_heads);
}

int launch_attn_step(cai_kv_s* kv, int layer, float* qkv, int64_t qkv_stride, int n_seq, int q_heads, int window,
                     float softcap, const float* theta, const int32_t* pos_dev, float* out, int64_t out_stride, int seq0)
{
  Context& c = ctx();
  if (layer < 0 || layer >= kv->n_layers) return set_error(CAI_ERR_INVALID, "attention: layer %d of %d", layer, kv->n_layers);
  if (n_seq < 1 || seq0 < 0 || seq0 + n_seq > kv->n_seq) return set_error(CAI_ERR_INVALID, "attention: %d sequences, cache holds %d", n_seq, kv->n_seq);
  if (q_heads % kv->kv_heads) return set_error(CAI_ERR_INVALID, "attention: %d query heads not a multiple of %d KV heads", q_heads, kv->kv_heads);
  if (q_heads > kv->part_q_heads) return set_error(CAI_ERR_INVALID, "attention: %d query heads exceed the cache's scratch (%d)", q_heads, kv->part_q_heads);
  AttnParams p{};
  p.qkv = qkv; p.qkv_stride = qkv_stride; p.kc = kv->k; p.vc = kv->v;
  p.seq_elems = kv->seq_elems(); p.layer_off = (int64_t)layer * kv->layer_elems();
  p.q_heads = q_heads; p.kv_heads = kv->kv_heads; p.hd = kv->head_dim; p.max_ctx = kv->max_ctx;
  p.window = window; p.softcap = softcap; p.inv_sqrt = 1.0f / sqrtf((float)kv->head_dim);
  p.theta = theta; p.pos = pos_dev; p.split_len = kv->split_len; p.n_splits = kv->n_splits;
  p.part = kv->part; p.out = out; p.out_stride = out_stride; p.seq0 = seq0;
  p.counters = kv->d_counters;
  if (kv->dtype == CAI_KV_F16) return launch_split_g<__half>(p, n_seq, c.stream);
  return launch_split_g<float>(p, n_seq, c.stream);
}

// ------------------------------------------------------------------------------------------
// cache lifetime
// ------------------------------------------------------------------------------------------
int kv_alloc(cai_kv_s* kv, int n_seq, int n_layers, int kv_heads, int head_dim, int max_ctx, int dtype)
{
  if (n_seq < 1 || n_layers < 1 || kv_heads < 1 || head_dim < 2 || (head_dim & 1) || head_dim > 128 || max_ctx < 1)
    return set_error(CAI_ERR_INVALID, "kv cache: bad geometry seq=%d layers=%d kv_heads=%d head_dim=%d max_ctx=%d", n_seq, n_layers, kv_heads, head_dim, max_ctx);
  if (dtype != CAI_KV_F32 && dtype != CAI_KV_F16) return set_error(CAI_ERR_INVALID, "kv cache: dtype %d", dtype);
  kv->n_seq = n_seq; kv->n_layers = n_layers; kv->kv_heads = kv_heads; kv->head_dim = head_dim; kv->max_ctx = max_ctx; kv->dtype = dtype;
  kv->len.assign((size_t)n_seq * n_layers, 0);
  int sl = (max_ctx + 47) / 48; sl = (sl + 31) / 32 * 32; if (sl < 32) sl = 32;
  kv->split_len = sl; kv->n_splits = (max_ctx + sl - 1) / sl;   // <= 48 by construction (the merge stage holds 64)
  const size_t bytes = (size_t)kv->seq_elems() * n_seq * kv->elem();
  CAI_HIP(hipMalloc(&kv->k, bytes));
  CAI_HIP(hipMalloc(&kv->v, bytes));
  CAI_HIP(hipMemsetAsync(kv->k, 0, bytes, ctx().stream));
  CAI_HIP(hipMemsetAsync(kv->v, 0, bytes, ctx().stream));
  kv->part_q_heads = kv_heads * 8;
  CAI_HIP(hipMalloc(&kv->part, (size_t)n_seq * kv->part_q_heads * kv->n_splits * (head_dim + 2) * sizeof(float)));
  CAI_HIP(hipMalloc(&kv->d_len, sizeof(int32_t) * n_seq));
  CAI_HIP(hipMalloc(&kv->d_counters, sizeof(int) * n_seq * kv_heads));
  CAI_HIP(hipMemsetAsync(kv->d_counters, 0, sizeof(int) * n_seq * kv_heads, ctx().stream));
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  return CAI_OK;
}

void kv_free(cai_kv_s* kv)
{
  if (kv->k) (void)hipFree(kv->k);
  if (kv->v) (void)hipFree(kv->v);
  if (kv->part) (void)hipFree(kv->part);
  if (kv->d_len) (void)hipFree(kv->d_len);
  if (kv->d_counters) (void)hipFree(kv->d_counters);
  kv->d_counters = nullptr;
  kv->k = kv->v = nullptr; kv->part = nullptr; kv->d_len = nullptr;
}

// Deep copy of the live rows of one sequence (TNNetDecoderSessionSnapshot, neural/neuraldecode.pas:1089-1142).
int kv_snapshot(cai_kv_s* kv, int seq, cai_kv_snap_s** out)
{
  cai_kv_snap_s* s = new cai_kv_snap_s();
  s->n_layers = kv->n_layers; s->kv_heads = kv->kv_heads; s->head_dim = kv->head_dim; s->dtype = kv->dtype;
  s->len.resize(kv->n_layers);
  int rows = 0;
  for (int l = 0; l < kv->n_layers; l++) { s->len[l] = kv->len_at(seq, l); rows = std::max(rows, s->len[l]); }
  s->rows = rows;
  if (rows > 0) {
    const size_t bytes = (size_t)kv->n_layers * kv->kv_heads * rows * kv->head_dim * kv->elem();
    if (hipMalloc(&s->k, bytes) != hipSuccess || hipMalloc(&s->v, bytes) != hipSuccess) {
      if (s->k) (void)hipFree(s->k);
      delete s; return set_error(CAI_ERR_NOMEM, "kv snapshot: out of device memory (%zu bytes)", 2 * bytes);
    }
    const size_t row_b = (size_t)kv->head_dim * kv->elem();
    for (int which = 0; which < 2; which++) {
      const char* src = (const char*)(which ? kv->v : kv->k) + (size_t)seq * kv->seq_elems() * kv->elem();
      char* dst = (char*)(which ? s->v : s->k);
      // [layer*kv_heads] planes of max_ctx rows -> planes of `rows` rows
      CAI_HIP(hipMemcpy2DAsync(dst, (size_t)rows * row_b, src, (size_t)kv->max_ctx * row_b, (size_t)rows * row_b,
                               (size_t)kv->n_layers * kv->kv_heads, hipMemcpyDeviceToDevice, ctx().stream));
    }
    CAI_HIP(hipStreamSynchronize(ctx().stream));
  }
  *out = s;
  return CAI_OK;
}

int kv_restore(cai_kv_s* kv, int seq, const cai_kv_snap_s* s)
{
  if (s->n_layers != kv->n_layers || s->kv_heads != kv->kv_heads || s->head_dim != kv->head_dim)
    return set_error(CAI_ERR_INVALID, "kv restore: snapshot geometry differs from the cache");
  if (s->dtype != kv->dtype) return set_error(CAI_ERR_INVALID, "kv restore: snapshot element type differs from the cache (mode must match)");
  if (s->rows > kv->max_ctx) return set_error(CAI_ERR_INVALID, "kv restore: snapshot holds %d rows, cache %d", s->rows, kv->max_ctx);
  if (s->rows > 0) {
    const size_t row_b = (size_t)kv->head_dim * kv->elem();
    for (int which = 0; which < 2; which++) {
      char* dst = (char*)(which ? kv->v : kv->k) + (size_t)seq * kv->seq_elems() * kv->elem();
      const char* src = (const char*)(which ? s->v : s->k);
      CAI_HIP(hipMemcpy2DAsync(dst, (size_t)kv->max_ctx * row_b, src, (size_t)s->rows * row_b, (size_t)s->rows * row_b,
                               (size_t)kv->n_layers * kv->kv_heads, hipMemcpyDeviceToDevice, ctx().stream));
    }
    CAI_HIP(hipStreamSynchronize(ctx().stream));
  }
  for (int l = 0; l < kv->n_layers; l++) kv->len_at(seq, l) = s->len[l];
  return CAI_OK;
}

}  // namespace cai

// ------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------
using namespace cai;

extern "C" int cai_kv_create(int n_layers, int kv_heads, int head_dim, int max_ctx, int kv_dtype, cai_kv_t* out)
{
  CAI_READY();
  CAI_REQUIRE(out, "cai_kv_create: null out");
  cai_kv_s* kv = new cai_kv_s();
  const int rc = kv_alloc(kv, 1, n_layers, kv_heads, head_dim, max_ctx, kv_dtype);
  if (rc) { kv_free(kv); delete kv; return rc; }
  *out = kv;
  return CAI_OK;
}

extern "C" int cai_kv_destroy(cai_kv_t kv)
{
  if (!kv) return CAI_OK;
  (void)hipStreamSynchronize(ctx().stream);
  kv_free(kv); delete kv;
  return CAI_OK;
}

extern "C" int cai_kv_reset(cai_kv_t kv)
{
  CAI_REQUIRE(kv, "cai_kv_reset: null cache");
  std::fill(kv->len.begin(), kv->len.end(), 0);
  return CAI_OK;
}

extern "C" int cai_kv_truncate(cai_kv_t kv, int n)
{
  CAI_REQUIRE(kv, "cai_kv_truncate: null cache");
  CAI_REQUIRE(n >= 0, "cai_kv_truncate: negative length %d", n);
  for (auto& l : kv->len) if (l > n) l = n;
  return CAI_OK;
}

extern "C" int cai_kv_len(cai_kv_t kv, int layer, int* len_out)
{
  CAI_REQUIRE(kv && len_out, "cai_kv_len: null argument");
  CAI_REQUIRE(layer >= 0 && layer < kv->n_layers, "cai_kv_len: layer %d of %d", layer, kv->n_layers);
  *len_out = kv->len_at(0, layer);
  return CAI_OK;
}

extern "C" int cai_kv_snapshot(cai_kv_t kv, cai_kv_snap_t* out)
{
  CAI_READY();
  CAI_REQUIRE(kv && out, "cai_kv_snapshot: null argument");
  return kv_snapshot(kv, 0, out);
}

extern "C" int cai_kv_restore(cai_kv_t kv, cai_kv_snap_t snap)
{
  CAI_READY();
  CAI_REQUIRE(kv && snap, "cai_kv_restore: null argument");
  return kv_restore(kv, 0, snap);
}

extern "C" int cai_kv_snap_destroy(cai_kv_snap_t s)
{
  if (!s) return CAI_OK;
  if (s->k) (void)hipFree(s->k);
  if (s->v) (void)hipFree(s->v);
  delete s;
  return CAI_OK;
}

extern "C" int cai_attn_decode(cai_kv_t kv, int layer, const float* qkv, int q_heads, int window, float softcap,
                               float* out, int flags)
{
  CAI_READY();
  CAI_REQUIRE(kv && qkv && out, "cai_attn_decode: null argument");
  CAI_REQUIRE(layer >= 0 && layer < kv->n_layers, "cai_attn_decode: layer %d of %d", layer, kv->n_layers);
  CAI_REQUIRE(q_heads > 0 && q_heads % kv->kv_heads == 0, "cai_attn_decode: %d query heads vs %d KV heads", q_heads, kv->kv_heads);
  Context& c = ctx();
  const int len = kv->len_at(0, layer);
  if (len >= kv->max_ctx) return set_error(CAI_ERR_STATE, "cai_attn_decode: cache full (%d rows)", kv->max_ctx);
  const int hd = kv->head_dim;
  const size_t in_b = (size_t)(q_heads + 2 * kv->kv_heads) * hd * sizeof(float), out_b = (size_t)q_heads * hd * sizeof(float);
  // the kernel rotates/append from a mutable row: always work on a private device copy
  int rc = ensure_stage(&c.stage_in, &c.stage_in_cap, in_b); if (rc) return rc;
  CAI_HIP(hipMemcpyAsync(c.stage_in, qkv, in_b, (flags & CAI_X_DEVICE) ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, c.stream));
  float* d_out = out;
  if (!(flags & CAI_Y_DEVICE)) { rc = ensure_stage(&c.stage_out, &c.stage_out_cap, out_b); if (rc) return rc; d_out = (float*)c.stage_out; }
  c.h_small[0] = len;
  CAI_HIP(hipMemcpyAsync(kv->d_len, c.h_small, sizeof(int32_t), hipMemcpyHostToDevice, c.stream));
  rc = launch_attn_step(kv, layer, (float*)c.stage_in, 0, 1, q_heads, window, softcap, nullptr, kv->d_len, d_out, 0, 0);
  if (rc) return rc;
  if (!(flags & CAI_Y_DEVICE)) CAI_HIP(hipMemcpyAsync(out, d_out, out_b, hipMemcpyDeviceToHost, c.stream));
  CAI_HIP(hipStreamSynchronize(c.stream));
  kv->len_at(0, layer) = len + 1;
  return CAI_OK;
}
