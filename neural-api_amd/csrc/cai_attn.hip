// KV cache + cached grouped-query decode attention for gfx950.
//
// Layer semantics (TNNetFusedSDPA; neural/neural.cl:2354-2499): the token row is [Q | K | V]; K and V are
// appended to a head-major cache (row (g, p) at (g*MaxCtx + p)*Dk), then for each query head h (KV head
// g = h / group) out_h = softmax(q_h . K_g / sqrt(Dk)) V_g over the live rows [jStart, len).
//
// Device formulation: split-K over the key axis; a slice of the live rows per work-group, a small second kernel
// (one work-group per query head) merges the slices.  (Merging inside the first kernel through an arrival counter was
// measured slower: every device-coherent hand-off between work-groups costs a memory round trip of ~2.5 us.)  RoPE of
// q and of the new k row and the cache append happen inside the split kernel.  Two split kernels:
//   attn_group_kernel       one work-group per (slice, KV head) serves the whole group of query heads, so K and V are
//                           fetched once; three phases per slice (scores -> LDS, softmax, value sum).  Used when the
//                           grid fills the chip by itself (long caches, several sequences, prompt ingestion).
//   attn_split_head_kernel  one work-group per (slice, QUERY head), online softmax in registers; the G heads of a
//                           group re-read the slice from L2.  G times more work-groups: the better one for one
//                           sequence with a short cache.
// Cache element types: fp32, IEEE half, or int8 codes with one fp32 scale per cached row (neural/neural.cl:2501-2687).
#include "cai_internal.hpp"
#include "cai_gemv_common.hpp"

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


// DS consecutive cache elements as floats with ONE vector load (the head width is a multiple of DS, so a lane's
// DS-wide slot is either wholly inside the row or wholly outside it)
template <int DS, typename KV_T> __device__ __forceinline__ void load_row_vec(const KV_T* src, float (&o)[DS]);
template <> __device__ __forceinline__ void load_row_vec<1, float>(const float* s, float (&o)[1]) { o[0] = s[0]; }
template <> __device__ __forceinline__ void load_row_vec<2, float>(const float* s, float (&o)[2]) { const float2 v = *reinterpret_cast<const float2*>(s); o[0] = v.x; o[1] = v.y; }
template <> __device__ __forceinline__ void load_row_vec<4, float>(const float* s, float (&o)[4]) { const float4 v = *reinterpret_cast<const float4*>(s); o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }
template <> __device__ __forceinline__ void load_row_vec<1, __half>(const __half* s, float (&o)[1]) { o[0] = __half2float(s[0]); }
template <> __device__ __forceinline__ void load_row_vec<2, __half>(const __half* s, float (&o)[2]) { const __half2 v = *reinterpret_cast<const __half2*>(s); o[0] = __low2float(v); o[1] = __high2float(v); }
template <> __device__ __forceinline__ void load_row_vec<4, __half>(const __half* s, float (&o)[4])
{
  const uint2 r = *reinterpret_cast<const uint2*>(s);
  const __half2 a = __builtin_bit_cast(__half2, r.x), b = __builtin_bit_cast(__half2, r.y);
  o[0] = __low2float(a); o[1] = __high2float(a); o[2] = __low2float(b); o[3] = __high2float(b);
}

template <> __device__ __forceinline__ void load_row_vec<1, int8_t>(const int8_t* s, float (&o)[1]) { o[0] = (float)s[0]; }
template <> __device__ __forceinline__ void load_row_vec<2, int8_t>(const int8_t* s, float (&o)[2])
{
  const int r = *reinterpret_cast<const short*>(s);
  o[0] = (float)(int8_t)(r & 0xff); o[1] = (float)(int8_t)((r >> 8) & 0xff);
}
template <> __device__ __forceinline__ void load_row_vec<4, int8_t>(const int8_t* s, float (&o)[4])
{
  const int r = *reinterpret_cast<const int*>(s);
  o[0] = (float)((r << 24) >> 24); o[1] = (float)((r << 16) >> 24); o[2] = (float)((r << 8) >> 24); o[3] = (float)(r >> 24);
}

// max over each half-wave (32 lanes), result in every lane of that half
__device__ __forceinline__ float half_wave_allmax(float v)
{
  for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// One cached row of an int8 cache from DS elements per lane of a half-wave (neural/neural.cl:2549-2578): the maximum
// over FINITE magnitudes, zero codes and unit scale when that maximum is zero or denormal, else scale = max / 127 and
// code = clamp(rint(v * (1/max) * 127)), NaN -> 0.  Lanes beyond the head width pass zeros.  On return v[] holds the
// codes as floats.
template <int DS> __device__ __forceinline__ float quantise_row_i8(float (&v)[DS])
{
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < DS; i++) {
    const float a = fabsf(v[i]);
    if (__builtin_bit_cast(uint32_t, a) <= 0x7F7FFFFFu) m = fmaxf(m, a);
  }
  m = half_wave_allmax(m);
  const bool usable = __builtin_bit_cast(uint32_t, m) >= 0x00800000u;
  const float recip = usable ? 1.0f / m : 0.0f;
#pragma unroll
  for (int i = 0; i < DS; i++) {
    float scaled = v[i] * recip * 127.0f;
    if (!usable || __builtin_bit_cast(uint32_t, fabsf(v[i])) > 0x7F800000u) scaled = 0.0f;
    v[i] = fminf(fmaxf(rintf(scaled), -127.0f), 127.0f);
  }
  return usable ? m / 127.0f : 1.0f;
}

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
  int seq_mul;                 // 1: activation row s uses cache sequence seq0 + s; 0: all rows share sequence seq0 (prompt)
  int appended;                // 1: the K,V rows of this step are already in the cache (prompt ingestion)
  float* part_override;        // split partials buffer when more rows than cache sequences are in flight
  float* ksc; float* vsc;      // int8 caches: row scales [seq][layer][kv_head][max_ctx]
  int64_t seq_rows, layer_row_off;
  int evict_sinks, evict_cap;  // cap > 0: only the first `sinks` positions and the latest cap - sinks stay cached
  const float* qn_gain; const float* kn_gain; float qk_eps;   // full-width RMSNorm of q and of k applied while they are read (null: rows are used as they are)
  unsigned* merge_cnt;         // decode steps: arrival counters [seq][head]; the work-group that completes the last slice merges (null: a merge launch follows)
  unsigned long long* timeline; // stamps of this launch's work-groups (null: none)
};

// ---- merge of the split partials inside the split kernels ----
// The slices of a head (or of a KV head's group of heads) finish in any order on any XCD.  Each work-group writes its partial
// through to memory (agent-scope stores: the XCDs' L2 caches are not coherent with one another inside a launch), waits for the
// stores to be acknowledged and then counts itself in; the one that counts last reads all partials back at agent scope and
// writes the finished rows.  The counter wraps to zero on the last arrival, so it needs no clearing between launches.  No
// cache-wide fence is involved (a __threadfence per work-group measured several times the merge launch it saves).
__device__ __forceinline__ void part_store(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float part_load(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Hand-over of the partial results.  The form built by default relies on what gfx942 / gfx950 do, not on the language's
// memory model: the partials are stored with agent-scope atomic stores (written through to memory, bypassing the
// non-coherent caches), vmcnt(0) returns only when those stores have been acknowledged, the work-group barrier orders every
// wave's acknowledgement before thread 0's agent-scope increment, and the last arriver reads with agent-scope atomic loads
// issued after the barrier that publishes s_is_last (atomic loads are not moved above it by the compiler).  It breaks if
// the partials are accessed with ordinary loads or stores, or on a target where an acknowledged agent-scope store may still
// be invisible to another compute unit.  -DCAI_MERGE_RELACQ builds the form the memory model guarantees (release increment,
// acquire fence in the last arriver); it writes back and invalidates the L2 of the XCD on every hand-over and takes the
// 7B batch-1 step from 1.52 to 1.60 ms.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(CAI_MERGE_RELACQ) && !defined(__gfx950__) && !defined(__gfx942__)
#error "merge_if_last: the relaxed hand-over is only valid on gfx942 / gfx950; build with -DCAI_MERGE_RELACQ"
#endif
// heads qh0 .. qh0 + n_heads - 1 of sequence `seq`; every thread of the work-group calls it after its partial stores
__device__ __forceinline__ void merge_if_last(const AttnParams& p, int seq, int qh0, int n_heads, int s_first, int n_active, int counter)
{
  __shared__ int s_is_last;
  __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): this thread's partial stores have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0)
#ifdef CAI_MERGE_RELACQ
    s_is_last = __builtin_amdgcn_atomic_inc32(p.merge_cnt + counter, (unsigned)n_active - 1, __ATOMIC_RELEASE, "agent") == (unsigned)n_active - 1;
#else
    s_is_last = __builtin_amdgcn_atomic_inc32(p.merge_cnt + counter, (unsigned)n_active - 1, __ATOMIC_RELAXED, "agent") == (unsigned)n_active - 1;
#endif
  __syncthreads();
  timeline_stamp(p.timeline, 6);
  if (!s_is_last) return;
#ifdef CAI_MERGE_RELACQ
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#endif
  // One round trip per MB slices: every thread requests, per slice, its value and the slice's maximum and sum together (the
  // latter two are the same addresses in all threads), then folds the slices in order with a running maximum.
  constexpr int MB = 12;
  const int hd = p.hd;
  for (int o = threadIdx.x; o < n_heads * hd; o += blockDim.x) {
    const int qh = qh0 + o / hd, d = o % hd;
    const float* pt = p.part + (((int64_t)seq * p.q_heads + qh) * p.n_splits + s_first) * (hd + 2);
    float A = 0.0f, L = 0.0f, M = -1e30f;
    for (int s0 = 0; s0 < n_active; s0 += MB) {
      float v[MB], ms[MB], ls[MB];
#pragma unroll
      for (int u = 0; u < MB; u++) {
        const float* ps = pt + (int64_t)min(s0 + u, n_active - 1) * (hd + 2);
        v[u] = part_load(ps + d); ms[u] = part_load(ps + hd); ls[u] = part_load(ps + hd + 1);
      }
#pragma unroll
      for (int u = 0; u < MB; u++) {
        if (s0 + u < n_active && ls[u] > 0.0f) {
          const float mn = fmaxf(M, ms[u]), c0 = expf(M - mn), c1 = expf(ms[u] - mn);
          A = fmaf(v[u], c1, A * c0); L = fmaf(ls[u], c1, L * c0); M = mn;
        }
      }
    }
    p.out[(int64_t)seq * p.out_stride + qh * hd + d] = L > 0.0f ? A * (1.0f / L) : 0.0f;
  }
}

// Where the row of stream position `pos` lives and which rows are live.  Without eviction: slot = pos, rows
// [j_start, pos] (j_start > 0 under a sliding window).  With sink + recent-window eviction (TNNetStreamingDecoder.
// EnableEviction, neural/neuraldecode.pas:1257-1276) the cache holds positions [0, sinks) and the latest cap - sinks;
// instead of shifting rows on every token the recent part is a ring: slot = sinks + (pos - sinks) mod (cap - sinks),
// and all cap rows are live.  Keys keep the rotation of their own position, the query that of `pos`.
struct LiveRows { int slot, len, j_start; };
__device__ __forceinline__ LiveRows live_rows(const AttnParams& p, int pos)
{
  LiveRows r;
  if (p.evict_cap > 0 && pos >= p.evict_cap) {
    r.slot = p.evict_sinks + (pos - p.evict_sinks) % (p.evict_cap - p.evict_sinks); r.len = p.evict_cap; r.j_start = 0;
  } else {
    r.slot = pos; r.len = pos + 1;
    r.j_start = (p.window > 0 && r.len > p.window) ? r.len - p.window : 0;
  }
  return r;
}

// ---- split kernel: RoPE (neural/neural.cl:1517-1542) + KV append (2354-2379) + one slice of the cached decode
//      (2406-2499), all query heads of a KV head in ONE work-group, so K and V are fetched once.
//
//      16 lanes x 8 elements cover a row, a wave holds 4 rows, the work-group 16 rows per pass; every load is 16
//      contiguous bytes per lane and a wave's load is 4 whole rows.  Three phases like the reference kernel, but per
//      slice: (1) scores of the slice into LDS (dot products reduced over 16 lanes with DPP), (2) slice maximum,
//      exp-shift and sum per head, (3) the value sum.  The query heads are taken HC at a time (q and the accumulators
//      live in registers: 8*HC each); a second chunk of heads re-reads the slice from cache.  The slice partial
//      (sum_j e_j V_j, max, sum e_j) goes to the merge kernel, or straight to the output when the live range fits one
//      slice. ----
template <typename KV_T> struct Row8;
template <> struct Row8<float>  { float4 a, b; };
template <> struct Row8<__half> { uint4 a; };
template <> struct Row8<int8_t> { uint2 a; };

__device__ __forceinline__ void load8(const float* s, Row8<float>& r) { r.a = reinterpret_cast<const float4*>(s)[0]; r.b = reinterpret_cast<const float4*>(s)[1]; }
__device__ __forceinline__ void load8(const __half* s, Row8<__half>& r) { r.a = *reinterpret_cast<const uint4*>(s); }
__device__ __forceinline__ void load8(const int8_t* s, Row8<int8_t>& r) { r.a = *reinterpret_cast<const uint2*>(s); }
__device__ __forceinline__ void unpack8(const Row8<float>& r, float (&v)[8])
{
  v[0] = r.a.x; v[1] = r.a.y; v[2] = r.a.z; v[3] = r.a.w; v[4] = r.b.x; v[5] = r.b.y; v[6] = r.b.z; v[7] = r.b.w;
}
__device__ __forceinline__ void unpack8(const Row8<__half>& r, float (&v)[8])
{
  const uint32_t w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
#pragma unroll
  for (int i = 0; i < 4; i++) { const __half2 h = __builtin_bit_cast(__half2, w[i]); v[2 * i] = __low2float(h); v[2 * i + 1] = __high2float(h); }
}
__device__ __forceinline__ void unpack8(const Row8<int8_t>& r, float (&v)[8])
{
  const int w[2] = {(int)r.a.x, (int)r.a.y};
#pragma unroll
  for (int i = 0; i < 2; i++) {
    v[4 * i] = (float)((w[i] << 24) >> 24); v[4 * i + 1] = (float)((w[i] << 16) >> 24);
    v[4 * i + 2] = (float)((w[i] << 8) >> 24); v[4 * i + 3] = (float)(w[i] >> 24);
  }
}

// wave64 maximum / sum in every lane: DPP steps inside the vector unit (row_shr within rows of 16, row_bcast15 / row_bcast31,
// total in lane 63, broadcast through a scalar register) instead of six trips through the LDS crossbar
__device__ __forceinline__ float wave_allmax(float v)
{
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, false)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x112, 0xf, 0xf, false)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, false)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, false)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false)));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_allsum(float v)
{
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wave_sum(v)), 63));
}
// gfx950 row swaps (a row = 16 lanes).  row_swap16: rows 1, 3 of x change places with rows 0, 2 of y, i.e. x = (x0 y0 x2 y2),
// y = (x1 y1 x3 y3); row_swap32: the upper half of x with the lower half of y, i.e. x = (x0 x1 y0 y1), y = (x2 x3 y2 y3).
// Written as instructions: through the builtins this compiler read BOTH results from the first register (sums came out as
// 2 x the first result).  The instruction needs two idle cycles after a vector write of its operands, which the compiler
// cannot see inside the statement: the s_nop provides them.
__device__ __forceinline__ void row_swap16(float& x, float& y) { asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x), "+v"(y)); }
__device__ __forceinline__ void row_swap32(float& x, float& y) { asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y)); }
// sum over each aligned group of 16 lanes, result in every lane of the group
__device__ __forceinline__ float row16_allsum(float v)
{
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xb1, 0xf, 0xf, true));   // lane ^ 1
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4e, 0xf, 0xf, true));   // lane ^ 2
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));  // 7 - lane within 8
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true));  // 15 - lane within 16
  return v;
}

template <int HC, typename KV_T, int NPF>     // NPF: passes in flight per lane
__global__ __launch_bounds__(256) void attn_group_kernel(const int32_t* hpos, const float* hqkv, const float* htheta, const long long hqkv_stride,
                                                         const int hheads, const int hgeo, const int hsl, const AttnParams p)
{
  // (leading scalar arguments arrive preloaded in scalar registers: position, q | k | v row and frequencies are requested without
  //  a round trip to the argument block; hheads = query heads | KV heads << 16, hgeo = slices | head width << 16, hsl = slice length)
  const unsigned long long tl0 = timeline_now();
  const int h_q_heads = hheads & 0xffff, h_kv_heads = hheads >> 16, h_n_splits = hgeo & 0xffff, h_hd = hgeo >> 16;
  extern __shared__ __align__(16) float lds[];
  constexpr bool I8 = sizeof(KV_T) == 1;
  const int G = h_q_heads / h_kv_heads, n_chunks = (G + HC - 1) / HC;
  const int split = blockIdx.x % h_n_splits, g = blockIdx.x / h_n_splits, seq = blockIdx.y;
  const int pos = hpos[seq];
  const LiveRows lr = live_rows(p, pos);
  const int len = lr.len, j_start = lr.j_start, slot = lr.slot;
  const int s_begin = max(j_start, split * hsl), s_end = min(len, (split + 1) * hsl);
  if (s_begin >= s_end) return;   // whole work-group leaves together, before any barrier
  const int s_first = j_start / hsl, s_last = (len - 1) / hsl;
  const int n_active = s_last - s_first + 1;
  const int n_rows = s_end - s_begin, n_pass = (n_rows + 15) >> 4;

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, r = lane >> 4, c = lane & 15, rr = 4 * w + r;
  const int hd = h_hd, qw = h_q_heads * hd, kw = h_kv_heads * hd, SL = hsl;
  const int d0 = 8 * c;
  const bool lane_on = d0 < hd;
  const int dl = lane_on ? d0 : 0;
  const float* row = hqkv + (int64_t)seq * hqkv_stride;
  const int64_t cache_seq = seq * p.seq_mul + p.seq0;
  KV_T* kc = reinterpret_cast<KV_T*>(p.kc) + cache_seq * p.seq_elems + p.layer_off + (int64_t)g * p.max_ctx * hd;
  KV_T* vc = reinterpret_cast<KV_T*>(p.vc) + cache_seq * p.seq_elems + p.layer_off + (int64_t)g * p.max_ctx * hd;
  float* ksc = nullptr; float* vsc = nullptr;
  if (I8) { const int64_t r0 = cache_seq * p.seq_rows + p.layer_row_off + (int64_t)g * p.max_ctx; ksc = p.ksc + r0; vsc = p.vsc + r0; }

  float* sq = lds;                          // rotated q [G][128]
  float* sS = sq + G * 128;                 // scores [G][SL]
  constexpr int PW = HC > 4 ? 8 : 4;
  float* sP = sS + G * SL;                  // softmax weights [chunk][SL][PW]
  float* sred = sP + n_chunks * SL * PW;    // per-wave value sums [4][HC][128]
  float* sML = sred + 4 * HC * 128;         // slice maximum [G], slice sum [G]

  Row8<KV_T> ring[NPF];
  float rsc[NPF];
  auto issue = [&](const KV_T* base, const float* scales, int slot, int t) {
    const int j = min(s_begin + 16 * t + rr, s_end - 1);
    load8(base + (int64_t)j * hd + dl, ring[slot]);     // lanes beyond the head width re-read its start; q is zero there
    if (I8) rsc[slot] = scales[j];
  };
  auto prime = [&](const KV_T* base, const float* scales) {
#pragma unroll
    for (int u = 0; u < NPF; u++) { rsc[u] = 0.0f; issue(base, scales, u, u); }   // (never conditional: passes beyond the slice re-read its last row, unused)
  };
  const bool owns_new = !p.appended && slot >= s_begin && slot < s_end;
  // Requests return in the order they were issued: the group's q pairs and frequencies (two turns of the work-group cover up to
  // eight 128-wide heads) go out first, the cached rows behind them, so that the rotation runs while the rows are on their way.
  const int n_qp = G * (hd >> 1);
  float qx0[2], qx1[2], qth[2];
#pragma unroll
  for (int u = 0; u < 2; u++) {
    const int e = min(tid + 256 * u, n_qp - 1), h = e / (hd >> 1), i = e % (hd >> 1);
    const float* qh = row + (g * G + h) * hd;
    qx0[u] = qh[2 * i]; qx1[u] = qh[2 * i + 1]; qth[u] = htheta ? htheta[i] : 0.0f;
  }
  if (!owns_new) prime(kc, ksc);
  timeline_put(p.timeline, 0, tl0);
  timeline_stamp(p.timeline, 1);

  // rotated q of the group's heads -> LDS
  for (int e = tid; e < n_qp; e += 256) {
    const int h = e / (hd >> 1), i = e % (hd >> 1);
    const int u = (e - tid) >> 8;
    float x0, x1, th;
    if (u < 2) { x0 = u ? qx0[1] : qx0[0]; x1 = u ? qx1[1] : qx1[0]; th = u ? qth[1] : qth[0]; }
    else { const float* qh = row + (g * G + h) * hd; x0 = qh[2 * i]; x1 = qh[2 * i + 1]; th = htheta ? htheta[i] : 0.0f; }
    if (htheta) {
      float sn, cs; sincosf((float)pos * th, &sn, &cs);
      const float y0 = cs * x0 - sn * x1, y1 = sn * x0 + cs * x1;
      x0 = y0; x1 = y1;
    }
    sq[h * 128 + 2 * i] = x0; sq[h * 128 + 2 * i + 1] = x1;
  }
  // the work-group whose slice holds `pos` appends the new row: wave 0, one half-wave each for K and V
  if (owns_new && w == 0) {
    const int l32 = lane & 31, is_v = lane >> 5, e0 = 4 * l32;
    const float* src = row + qw + (is_v ? kw : 0) + g * hd;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; i += 2) {
      const int d = e0 + i;
      float x0 = d < hd ? src[d] : 0.0f, x1 = d + 1 < hd ? src[d + 1] : 0.0f;
      if (htheta && !is_v && d < hd) {
        float sn, cs; sincosf((float)pos * htheta[d >> 1], &sn, &cs);
        const float y0 = cs * x0 - sn * x1, y1 = sn * x0 + cs * x1;
        x0 = y0; x1 = y1;
      }
      v[i] = x0; v[i + 1] = x1;
    }
    KV_T* dst = (is_v ? vc : kc) + (int64_t)slot * hd;
    if constexpr (I8) {
      const float scale = quantise_row_i8<4>(v);
#pragma unroll
      for (int i = 0; i < 4; i++) if (e0 + i < hd) dst[e0 + i] = (int8_t)v[i];
      if (l32 == 0) (is_v ? vsc : ksc)[slot] = scale;
    } else {
#pragma unroll
      for (int i = 0; i < 4; i++) if (e0 + i < hd) dst[e0 + i] = kv_from_float<KV_T>(v[i]);
    }
  }
  __syncthreads();      // q is staged; the appended row is visible to this work-group's loads
  if (owns_new) prime(kc, ksc);
  timeline_stamp(p.timeline, 4);

  // ---- phase 1: scores of the slice ----
  for (int ch = 0; ch < n_chunks; ch++) {
    const int h0 = ch * HC;
    if (ch > 0) prime(kc, ksc);
    float q[HC][8];
#pragma unroll
    for (int hh = 0; hh < HC; hh++)
#pragma unroll
      for (int i = 0; i < 8; i++) q[hh][i] = (lane_on && h0 + hh < G) ? sq[(h0 + hh) * 128 + d0 + i] : 0.0f;
    for (int t0 = 0; t0 < n_pass; t0 += NPF) {
#pragma unroll
      for (int u = 0; u < NPF; u++) {
        const int t = t0 + u;
        if (t < n_pass) {
          float v[8];
          unpack8(ring[u], v);
          const float rs = rsc[u];
          if (t + NPF < n_pass) issue(kc, ksc, u, t + NPF);
          float sv = 0.0f;
#pragma unroll
          for (int hh = 0; hh < HC; hh++) {
            float a = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) a = fmaf(q[hh][i], v[i], a);
            a = row16_allsum(a);
            if (c == hh) sv = a;
          }
          const int rl = 16 * t + rr;
          if (rl < n_rows && c < HC && h0 + c < G) {
            sS[(h0 + c) * SL + rl] = sv * (I8 ? rs * p.inv_sqrt : p.inv_sqrt);
          }
        }
      }
    }
  }
  prime(vc, vsc);        // the first value rows travel while the softmax runs
  __syncthreads();
  timeline_stamp(p.timeline, 5);

  // ---- phase 2: slice maximum, exp-shift and sum per head (wave w takes heads w, w+4, ..) ----
  for (int h = w; h < G; h += 4) {
    float m = -1e30f;
    if (p.softcap > 0.0f)
      for (int rl = lane; rl < n_rows; rl += 64) sS[h * SL + rl] = p.softcap * tanhf(sS[h * SL + rl] / p.softcap);
    for (int rl = lane; rl < n_rows; rl += 64) m = fmaxf(m, sS[h * SL + rl]);
    m = wave_allmax(m);
    float l = 0.0f;
    for (int rl = lane; rl < n_rows; rl += 64) {
      const float e = expf(sS[h * SL + rl] - m);
      l += e;
      sP[((h / HC) * SL + rl) * PW + h % HC] = I8 ? e * vsc[s_begin + rl] : e;
    }
    l = wave_allsum(l);
    if (lane == 0) { sML[h] = m; sML[G + h] = l; }
  }
  __syncthreads();

  timeline_stamp(p.timeline, 6);
  // ---- phase 3: value sums ----
  for (int ch = 0; ch < n_chunks; ch++) {
    const int h0 = ch * HC;
    if (ch > 0) prime(vc, vsc);
    float acc[HC][8];
#pragma unroll
    for (int hh = 0; hh < HC; hh++)
#pragma unroll
      for (int i = 0; i < 8; i++) acc[hh][i] = 0.0f;
    for (int t0 = 0; t0 < n_pass; t0 += NPF) {
#pragma unroll
      for (int u = 0; u < NPF; u++) {
        const int t = t0 + u;
        if (t < n_pass) {
          float v[8];
          unpack8(ring[u], v);
          if (t + NPF < n_pass) issue(vc, vsc, u, t + NPF);
          const int rl = 16 * t + rr;
          float pf[PW];
#pragma unroll
          for (int k4 = 0; k4 < PW; k4 += 4) {
            float4 pw = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (rl < n_rows) pw = *reinterpret_cast<const float4*>(sP + ((int64_t)ch * SL + rl) * PW + k4);
            pf[k4] = pw.x; pf[k4 + 1] = pw.y; pf[k4 + 2] = pw.z; pf[k4 + 3] = pw.w;
          }
#pragma unroll
          for (int hh = 0; hh < HC; hh++)
#pragma unroll
            for (int i = 0; i < 8; i++) acc[hh][i] = fmaf(pf[hh], v[i], acc[hh][i]);
        }
      }
    }
    // The wave's 4 row groups (rows of 16 lanes), then the 4 waves.  A transposing sum: the row-swap instructions of gfx950 turn
    // two registers into (row 0+1 | 2+3 of the first, of the second), then four into one whose row r holds the total of value
    // 4 q + r - (r0 + r1) + (r2 + r3) as a butterfly over lanes ^16, ^32 would give, in 1.5 instructions per value instead of
    // two LDS-crossbar permutes and two additions, and with one store per four values (the butterfly form took 3.8 of the
    // launch's 15 us at batch 8).
#pragma unroll
    for (int q4 = 0; q4 < 2 * HC; q4++) {
      float s2[2];
#pragma unroll
      for (int hf = 0; hf < 2; hf++) {
        const int n = 4 * q4 + 2 * hf;
        float x = acc[n >> 3][n & 7], y = acc[(n + 1) >> 3][(n + 1) & 7];
        row_swap16(x, y);
        s2[hf] = x + y;                 // rows: x0+x1 | y0+y1 | x2+x3 | y2+y3
      }
      row_swap32(s2[0], s2[1]);
      const float tot = s2[0] + s2[1];  // row r: total of value 4 q4 + r
      const int n = 4 * q4 + r;
      if (lane_on) sred[(w * HC + (n >> 3)) * 128 + d0 + (n & 7)] = tot;
    }
    __syncthreads();
    for (int o = tid; o < HC * hd; o += 256) {
      const int hh = o / hd, d = o % hd, h = h0 + hh;
      if (h < G) {
        const float A = (sred[(0 * HC + hh) * 128 + d] + sred[(1 * HC + hh) * 128 + d]) + (sred[(2 * HC + hh) * 128 + d] + sred[(3 * HC + hh) * 128 + d]);
        const float M = sML[h], Ls = sML[G + h];
        const int qh = g * G + h;
        if (n_active == 1) {
          p.out[(int64_t)seq * p.out_stride + qh * hd + d] = Ls > 0.0f ? A * (1.0f / Ls) : 0.0f;
        } else {
          float* pt = p.part + (((int64_t)seq * h_q_heads + qh) * h_n_splits + split) * (hd + 2);
          pt[d] = A;
          if (d == 0) { pt[hd] = M; pt[hd + 1] = Ls; }
        }
      }
    }
    __syncthreads();
  }
  timeline_stamp(p.timeline, 7);
}

// ---- the same split on the matrix cores: half-precision cache, 128-wide heads, groups of up to 16 query heads.
//      The VALU form above spends its time on instructions (8 conversions, 8 fused multiply-adds per head and a 4-step lane
//      reduction per head for every 16 bytes of K), one wave per SIMD.  Here a wave requests ALL its rows of the slice at once
//      (16-row tiles w, w + NW, ..: TPW tiles of K and of V, 16 KB in flight per wave) and the products are
//        S[row][head]  = K . q^T      v_mfma_f32_16x16x32_f16, K rows straight from memory as the A operand (lane = row,
//                                     16 bytes = 8 of the 32 contraction slots), q split hi + lo into two f16 planes in LDS;
//        O[head][dim] += P^T . V      the result registers of the first product (lane = head, 4 rows each of two tiles) ARE
//                                     the A operand of a 32-row step; P is scaled by 1024 and split hi + lo (its low part
//                                     stays clear of the f16 subnormal range); V goes through LDS as it arrives (row-major,
//                                     16-byte stores) and comes back as 32-bit words = two neighbouring dims of one row, so
//                                     that one byte permute per word pair builds the operand of the even and of the odd dims.
//      Every wave keeps its own maximum and sum per head; the four waves meet once, in LDS, and the slice partial has the
//      same form as above.  Same contract and tolerance as the VALU kernels (1e-5 against the oracle). ----
typedef _Float16 ph4_t __attribute__((ext_vector_type(4)));
typedef _Float16 ph8_t __attribute__((ext_vector_type(8)));
constexpr int GM_LD = 136;                         // halfs per staged row (128 + pad: 16-byte aligned, 4 rows apart = 16 banks apart)
constexpr int GM_FIXED = 2 * 16 * GM_LD * 2 + 512 + 1024;  // q hi | q lo | new K,V row | per-wave maximum and sum
constexpr int gm_lds_bytes(int tpw, int nw) { return GM_FIXED + nw * tpw * 16 * GM_LD * 2; }

// TPW 16-row tiles per wave, NW waves: 2 x 4 (slices of up to 128 rows) or 2 x 8 (up to 256: two waves per SIMD overlap each
// other's dependent LDS / matrix-core / soft-max chains)
// KV_T = int8_t: the codes become f16 exactly on their way into the operands (byte ^ 0x80 under a 0x64 exponent byte = 1152 + code,
// one packed subtraction: 1.25 instructions per element), the K row scale multiplies the finished score and the V row scale the
// soft-max weight before its hi + lo split, as in the VALU kernels (neural/neural.cl:2639-2640, 2683-2684).
__device__ __forceinline__ ph8_t gm_codes_to_halfs(uint32_t w0, uint32_t w1)
{
  typedef _Float16 gh2_t __attribute__((ext_vector_type(2)));
  const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u, K = 0x64646464u;
  const gh2_t off = {(_Float16)1152.0f, (_Float16)1152.0f};
  const gh2_t a = __builtin_bit_cast(gh2_t, __builtin_amdgcn_perm(K, x0, 0x04010400u)) - off, b = __builtin_bit_cast(gh2_t, __builtin_amdgcn_perm(K, x0, 0x04030402u)) - off;
  const gh2_t c = __builtin_bit_cast(gh2_t, __builtin_amdgcn_perm(K, x1, 0x04010400u)) - off, d = __builtin_bit_cast(gh2_t, __builtin_amdgcn_perm(K, x1, 0x04030402u)) - off;
  return ph8_t{a.x, a.y, b.x, b.y, c.x, c.y, d.x, d.y};
}
template <int TPW, int NW, typename KV_T>
__global__ __launch_bounds__(64 * NW) void attn_group_mfma_kernel(const int32_t* hpos, const float* hqkv, const float* htheta, const long long hqkv_stride,
                                                              const int hheads, const int hgeo, const int hsl, const AttnParams p)
{
  const unsigned long long tl0 = timeline_now();
  const int h_q_heads = hheads & 0xffff, h_kv_heads = hheads >> 16, h_n_splits = hgeo & 0xffff;
  constexpr int hd = 128;
  constexpr bool I8 = sizeof(KV_T) == 1;
  extern __shared__ __align__(16) unsigned char glds[];
  _Float16* sqh = reinterpret_cast<_Float16*>(glds);
  _Float16* sql = sqh + 16 * GM_LD;
  _Float16* snew = sql + 16 * GM_LD;                           // [K | V][128] (int8: the codes as bytes, then the two row scales at byte 256)
  float* sML = reinterpret_cast<float*>(snew + 256);           // [wave][head][maximum, sum]
  constexpr int REGION = TPW * 16 * GM_LD * 2;                 // bytes of a wave's V tiles (later: its [head][128] float sums)
  const int G = h_q_heads / h_kv_heads;
  const int split = blockIdx.x % h_n_splits, g = blockIdx.x / h_n_splits, seq = blockIdx.y;
  const int pos = hpos[seq];
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, n16 = lane & 15, kg = lane >> 4;
  const int qw = h_q_heads * hd, kw = h_kv_heads * hd;
  const float* row = hqkv + (int64_t)seq * hqkv_stride;
  // the group's q pairs and frequencies do not depend on the position: requested behind it, before anything waits
  float qx0[2], qx1[2], qth[2];
#pragma unroll
  for (int u = 0; u < 2; u++) {
    const int e = tid + 64 * NW * u, h = min(e >> 6, G - 1), i = e & 63;
    const float* qh = row + (g * G + h) * hd;
    qx0[u] = qh[2 * i]; qx1[u] = qh[2 * i + 1]; qth[u] = htheta ? htheta[i] : 0.0f;
  }
  const int SL = hsl, base = split * SL;
  const int64_t cache_seq = seq * p.seq_mul + p.seq0;
  KV_T* kc = reinterpret_cast<KV_T*>(p.kc) + cache_seq * p.seq_elems + p.layer_off + (int64_t)g * p.max_ctx * hd;
  KV_T* vc = reinterpret_cast<KV_T*>(p.vc) + cache_seq * p.seq_elems + p.layer_off + (int64_t)g * p.max_ctx * hd;
  float* ksc = nullptr; float* vsc = nullptr;
  if (I8) { const int64_t r0 = cache_seq * p.seq_rows + p.layer_row_off + (int64_t)g * p.max_ctx; ksc = p.ksc + r0; vsc = p.vsc + r0; }
  // contraction slots of a lane group: half cache dims 32 s + 8 kg .., int8 cache dims 32 kg + 8 s .. (a lane's 32 codes of a row are
  // two 16-byte requests)
  constexpr int KCH = I8 ? 2 : 4;          // 16-byte requests per lane and K tile
  // The wave's first K tile is requested before the position is known (its rows exist whatever the position: the slice lies
  // inside the cache; rows past the live range are masked), so the stream starts while the position is still on its way.
  uint4 kreg[TPW][4], vreg[TPW][4];
  {
    const int j = min(base + 16 * w + n16, p.max_ctx - 1);
#pragma unroll
    for (int s4 = 0; s4 < KCH; s4++) kreg[0][s4] = *reinterpret_cast<const uint4*>(kc + (int64_t)j * hd + (I8 ? 32 * kg + 16 * s4 : 32 * s4 + 8 * kg));
  }
  const LiveRows lr = live_rows(p, pos);
  const int len = lr.len, j_start = lr.j_start, slot = lr.slot;
  const int s_begin = max(j_start, base), s_end = min(len, base + SL);
  if (s_begin >= s_end) return;   // whole work-group leaves together, before any barrier
  const int s_first = j_start / SL, s_last = (len - 1) / SL;
  const int n_active = s_last - s_first + 1;

  // the work-group whose slice holds `pos` appends the new row (wave 0, one half-wave each for K and V): its raw elements are
  // requested here, in front of the cached rows (requests return in order)
  const bool owns_new = !p.appended && slot >= s_begin && slot < s_end;
  float nraw[4] = {0.0f, 0.0f, 0.0f, 0.0f}, nth[2] = {0.0f, 0.0f};
  if (owns_new && w == 0) {
    const int l32 = lane & 31, is_v = lane >> 5, e0 = 4 * l32;
    const float* src = row + qw + (is_v ? kw : 0) + g * hd + e0;
#pragma unroll
    for (int i = 0; i < 4; i++) nraw[i] = src[i];
    if (htheta) { nth[0] = htheta[e0 >> 1]; nth[1] = htheta[(e0 >> 1) + 1]; }
  }
  // int8: the scales of the rows whose scores this lane will hold (rows 4 kg .. 4 kg + 3 of every tile), in front of the rows
  float ks4[TPW][4], vs4[TPW][4];
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int j = min(base + 16 * (w + NW * t) + 4 * kg + i, s_end - 1);
      ks4[t][i] = I8 ? ksc[j] : 1.0f; vs4[t][i] = I8 ? vsc[j] : 1.0f;
    }
  // every other row of the wave's tiles, K first (the first product starts while V is still on its way).
  // Rows past the live range repeat its last row and are masked below.
#pragma unroll
  for (int t = 1; t < TPW; t++) {
    const int j = min(base + 16 * (w + NW * t) + n16, s_end - 1);
#pragma unroll
    for (int s4 = 0; s4 < KCH; s4++) kreg[t][s4] = *reinterpret_cast<const uint4*>(kc + (int64_t)j * hd + (I8 ? 32 * kg + 16 * s4 : 32 * s4 + 8 * kg));
  }
  // V rows as they lie in memory: half cache 4 rows x 256 bytes per request, int8 cache 8 rows x 128 bytes
  constexpr int VCH = I8 ? 2 : 4, VROWS = I8 ? 8 : 4;
  const int vrow = I8 ? lane >> 3 : kg, vcol = I8 ? 16 * (lane & 7) : 8 * n16;
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int i = 0; i < VCH; i++) {
      const int j = min(base + 16 * (w + NW * t) + VROWS * i + vrow, s_end - 1);
      vreg[t][i] = *reinterpret_cast<const uint4*>(vc + (int64_t)j * hd + vcol);
    }
  timeline_put(p.timeline, 0, tl0);
  timeline_stamp(p.timeline, 1);

  // rotated q of the group's heads as two f16 planes in LDS (wave w takes heads w, w + NW, ..; rows G .. 15 are zero)
#pragma unroll
  for (int u = 0; u < 16 / NW; u++) {
    const int h = w + NW * u, i = lane;
    _Float16 h0 = 0, h1 = 0, l0 = 0, l1 = 0;
    if (h < G) {
      float x0, x1, th;
      if (u < 2) { x0 = qx0[u]; x1 = qx1[u]; th = qth[u]; }
      else { const float* qh = row + (g * G + h) * hd; x0 = qh[2 * i]; x1 = qh[2 * i + 1]; th = htheta ? htheta[i] : 0.0f; }
      if (htheta) {
        float sn, cs; sincosf((float)pos * th, &sn, &cs);
        const float y0 = cs * x0 - sn * x1, y1 = sn * x0 + cs * x1;
        x0 = y0; x1 = y1;
      }
      split_f16(x0, h0, l0); split_f16(x1, h1, l1);
    }
    sqh[h * GM_LD + 2 * i] = h0; sqh[h * GM_LD + 2 * i + 1] = h1;
    sql[h * GM_LD + 2 * i] = l0; sql[h * GM_LD + 2 * i + 1] = l1;
  }
  // the new row: rotated, rounded to the cache's precision (int8: quantised, neural/neural.cl:2501-2580), stored, and kept in LDS for
  // this work-group's own products (its requests for that row went out before the store)
  if (owns_new && w == 0) {
    const int l32 = lane & 31, is_v = lane >> 5, e0 = 4 * l32;
    KV_T* dst = (is_v ? vc : kc) + (int64_t)slot * hd;
    float v4[4];
#pragma unroll
    for (int i = 0; i < 4; i += 2) {
      float x0 = nraw[i], x1 = nraw[i + 1];
      if (htheta && !is_v) {
        float sn, cs; sincosf((float)pos * nth[i >> 1], &sn, &cs);
        const float y0 = cs * x0 - sn * x1, y1 = sn * x0 + cs * x1;
        x0 = y0; x1 = y1;
      }
      v4[i] = x0; v4[i + 1] = x1;
    }
    if constexpr (I8) {
      const float scale = quantise_row_i8<4>(v4);
      int8_t* sb = reinterpret_cast<int8_t*>(snew);
#pragma unroll
      for (int i = 0; i < 4; i++) { dst[e0 + i] = (int8_t)v4[i]; sb[is_v * 128 + e0 + i] = (int8_t)v4[i]; }
      if (l32 == 0) { (is_v ? vsc : ksc)[slot] = scale; reinterpret_cast<float*>(snew + 128)[is_v] = scale; }
    } else {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const __half r = __float2half_rn(v4[i]);
        dst[e0 + i] = r; snew[is_v * 128 + e0 + i] = __builtin_bit_cast(_Float16, r);
      }
    }
  }
  __syncthreads();
  timeline_stamp(p.timeline, 4);

  ph8_t qh8[4], ql8[4];
#pragma unroll
  for (int s4 = 0; s4 < 4; s4++) {
    qh8[s4] = *reinterpret_cast<const ph8_t*>(sqh + n16 * GM_LD + (I8 ? 32 * kg + 8 * s4 : 32 * s4 + 8 * kg));
    ql8[s4] = *reinterpret_cast<const ph8_t*>(sql + n16 * GM_LD + (I8 ? 32 * kg + 8 * s4 : 32 * s4 + 8 * kg));
  }
  if (owns_new) {
    // the new row from LDS in place of what memory held; rows past the live range may be memory that was never written (the
    // new row's slot before this step): their V registers are cleared, 0 x NaN would poison the sums
    const int rs = slot - base;
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      const int r0 = 16 * (w + NW * t);
      if (rs >= r0 && rs < r0 + 16) {
        const unsigned char* sb = reinterpret_cast<const unsigned char*>(snew);
        if (n16 == rs - r0) {
#pragma unroll
          for (int s4 = 0; s4 < KCH; s4++) kreg[t][s4] = *reinterpret_cast<const uint4*>(sb + (I8 ? 32 * kg + 16 * s4 : 2 * (32 * s4 + 8 * kg)));
        }
#pragma unroll
        for (int i = 0; i < VCH; i++)
          if (VROWS * i + vrow == rs - r0) vreg[t][i] = *reinterpret_cast<const uint4*>(sb + (I8 ? 128 + vcol : 2 * (128 + vcol)));
        if (I8) {
#pragma unroll
          for (int i = 0; i < 4; i++)
            if (4 * kg + i == rs - r0) { ks4[t][i] = reinterpret_cast<const float*>(snew + 128)[0]; vs4[t][i] = reinterpret_cast<const float*>(snew + 128)[1]; }
        }
      }
#pragma unroll
      for (int i = 0; i < VCH; i++)
        if (base + r0 + VROWS * i + vrow >= s_end) vreg[t][i] = make_uint4(0u, 0u, 0u, 0u);
    }
  }

  // ---- scores of the wave's rows, maximum, weights ----
  typedef float gf4_t __attribute__((ext_vector_type(4)));
  gf4_t C[TPW];
#pragma unroll
  for (int t = 0; t < TPW; t++) {
    C[t] = gf4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s4 = 0; s4 < 4; s4++) {
      ph8_t a;
      if constexpr (I8) {
        const uint4 kq = kreg[t][s4 >> 1];
        a = (s4 & 1) ? gm_codes_to_halfs(kq.z, kq.w) : gm_codes_to_halfs(kq.x, kq.y);
      } else a = __builtin_bit_cast(ph8_t, kreg[t][s4]);
      C[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qh8[s4], C[t], 0, 0, 0);
      C[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, ql8[s4], C[t], 0, 0, 0);
    }
  }
  // lane (n16, kg) holds head n16 of rows 4 kg .. 4 kg + 3 of every tile
  float m_w = -1e30f;
  bool ok[TPW][4];
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int j = base + 16 * (w + NW * t) + 4 * kg + i;
      float sc = C[t][i] * (I8 ? ks4[t][i] * p.inv_sqrt : p.inv_sqrt);
      if (p.softcap > 0.0f) sc = p.softcap * tanhf(sc / p.softcap);
      ok[t][i] = j >= s_begin && j < s_end;
      C[t][i] = sc;
      if (ok[t][i]) m_w = fmaxf(m_w, sc);
    }
  m_w = fmaxf(m_w, __shfl_xor(m_w, 16, 64));
  m_w = fmaxf(m_w, __shfl_xor(m_w, 32, 64));
  float l_w = 0.0f;
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int i = 0; i < 4; i++) { C[t][i] = ok[t][i] ? expf(C[t][i] - m_w) : 0.0f; l_w += C[t][i]; }
  l_w += __shfl_xor(l_w, 16, 64);
  l_w += __shfl_xor(l_w, 32, 64);
  timeline_stamp(p.timeline, 5);

  // ---- value sums ----
  unsigned char* region = glds + GM_FIXED + w * REGION;
  _Float16* sV = reinterpret_cast<_Float16*>(region);
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int i = 0; i < VCH; i++) {
      if constexpr (I8) {
        const uint4 vq = vreg[t][i];
        _Float16* dstv = sV + (16 * t + 8 * i + vrow) * GM_LD + vcol;
        *reinterpret_cast<ph8_t*>(dstv) = gm_codes_to_halfs(vq.x, vq.y);
        *reinterpret_cast<ph8_t*>(dstv + 8) = gm_codes_to_halfs(vq.z, vq.w);
      } else *reinterpret_cast<uint4*>(sV + (16 * t + 4 * i + kg) * GM_LD + 8 * n16) = vreg[t][i];
    }
  gf4_t Oe[4], Oo[4];
#pragma unroll
  for (int u = 0; u < 4; u++) { Oe[u] = gf4_t{0.0f, 0.0f, 0.0f, 0.0f}; Oo[u] = gf4_t{0.0f, 0.0f, 0.0f, 0.0f}; }
#pragma unroll
  for (int b = 0; b < TPW / 2; b++) {
    // contraction slot e of this lane group = row 4 kg + (e & 3) of tile 2 b + (e >> 2), in both operands
    ph8_t ph, pl;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int t = 2 * b + (e >> 2), i = e & 3;
      const float pe = I8 ? (ok[t][i] ? C[t][i] * vs4[t][i] : 0.0f) : C[t][i];      // (a dead row's scale is whatever memory holds)
      _Float16 hv, lv; split_f16(pe * 1024.0f, hv, lv); ph[e] = hv; pl[e] = lv;
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      uint32_t wv[8];
#pragma unroll
      for (int e = 0; e < 8; e++)
        wv[e] = *reinterpret_cast<const uint32_t*>(sV + (16 * (2 * b + (e >> 2)) + 4 * kg + (e & 3)) * GM_LD + 32 * u + 2 * n16);
      uint4 va, vb;       // column n16 of the even dims 32 u + 2 n16 and of the odd dims 32 u + 2 n16 + 1
      va.x = __builtin_amdgcn_perm(wv[1], wv[0], 0x05040100u); vb.x = __builtin_amdgcn_perm(wv[1], wv[0], 0x07060302u);
      va.y = __builtin_amdgcn_perm(wv[3], wv[2], 0x05040100u); vb.y = __builtin_amdgcn_perm(wv[3], wv[2], 0x07060302u);
      va.z = __builtin_amdgcn_perm(wv[5], wv[4], 0x05040100u); vb.z = __builtin_amdgcn_perm(wv[5], wv[4], 0x07060302u);
      va.w = __builtin_amdgcn_perm(wv[7], wv[6], 0x05040100u); vb.w = __builtin_amdgcn_perm(wv[7], wv[6], 0x07060302u);
      const ph8_t a8 = __builtin_bit_cast(ph8_t, va), b8 = __builtin_bit_cast(ph8_t, vb);
      Oe[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ph, a8, Oe[u], 0, 0, 0);
      Oe[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pl, a8, Oe[u], 0, 0, 0);
      Oo[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ph, b8, Oo[u], 0, 0, 0);
      Oo[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pl, b8, Oo[u], 0, 0, 0);
    }
  }
  timeline_stamp(p.timeline, 6);
  // ---- meeting of the waves: lane (n16, kg) holds heads 4 kg .. 4 kg + 3, dims 32 u + 2 n16 (+ 1) ----
  float* sO = reinterpret_cast<float*>(region);       // [head][128], over the wave's own V tiles (all read by now)
#pragma unroll
  for (int i = 0; i < 4; i++)
    if (4 * kg + i < G) {
#pragma unroll
      for (int u = 0; u < 4; u++) *reinterpret_cast<float2*>(sO + (4 * kg + i) * 128 + 32 * u + 2 * n16) = make_float2(Oe[u][i], Oo[u][i]);
    }
  if (kg == 0) { sML[(w * 16 + n16) * 2] = m_w; sML[(w * 16 + n16) * 2 + 1] = l_w; }
  __syncthreads();
  for (int o = tid; o < G * hd; o += 64 * NW) {
    const int h = o >> 7, d = o & 127;
    float mw[NW], lw[NW], ow[NW];
#pragma unroll
    for (int k = 0; k < NW; k++) {
      mw[k] = sML[(k * 16 + h) * 2]; lw[k] = sML[(k * 16 + h) * 2 + 1];
      ow[k] = reinterpret_cast<const float*>(glds + GM_FIXED + k * REGION)[h * 128 + d];
    }
    float M = mw[0];
#pragma unroll
    for (int k = 1; k < NW; k++) M = fmaxf(M, mw[k]);
    float A = 0.0f, Ls = 0.0f;
#pragma unroll
    for (int k4 = 0; k4 < NW; k4 += 4) {      // fixed order: groups of four waves
      float e[4];
#pragma unroll
      for (int k = 0; k < 4; k++) e[k] = lw[k4 + k] > 0.0f ? expf(mw[k4 + k] - M) : 0.0f;
      A += (ow[k4] * e[0] + ow[k4 + 1] * e[1]) + (ow[k4 + 2] * e[2] + ow[k4 + 3] * e[3]);
      Ls += (lw[k4] * e[0] + lw[k4 + 1] * e[1]) + (lw[k4 + 2] * e[2] + lw[k4 + 3] * e[3]);
    }
    A *= 1.0f / 1024.0f;
    const int qh = g * G + h;
    if (n_active == 1) {
      p.out[(int64_t)seq * p.out_stride + qh * hd + d] = Ls > 0.0f ? A * (1.0f / Ls) : 0.0f;
    } else {
      float* pt = p.part + (((int64_t)seq * h_q_heads + qh) * h_n_splits + split) * (hd + 2);
      pt[d] = A;
      if (d == 0) { pt[hd] = M; pt[hd + 1] = Ls; }
    }
  }
  timeline_stamp(p.timeline, 7);
}

// ---- merge of the split partials: one work-group per query head.  Four quarter-groups of head_dim threads each take every
//      fourth slice (all their loads go out together: one round trip for up to 32 slices per quarter), fold them with a running
//      maximum, and meet in LDS. ----
template <int MR>      // slices per quarter and round trip: 12, or 32 for long caches (130k rows = 508 slices: 4 dependent rounds instead of 11)
__global__ __launch_bounds__(512) void attn_merge_kernel(const int32_t* hpos, const float* hpart, float* hout, const long long hout_stride,
                                                         const int hheads, const int hgeo, const int hsl, const AttnParams p)
{
  const int h_q_heads = hheads & 0xffff, h_n_splits = hgeo & 0xffff, h_hd = hgeo >> 16;     // (preloaded leading arguments, as in the split kernels)
  const int qh = blockIdx.x, seq = blockIdx.y;
  const int hd = h_hd;
  __shared__ float qA[4][128], qM[4], qL[4];
  const int quarter = threadIdx.x >> 7, d = threadIdx.x & 127;
  // Without a sliding window the first live slice is slice 0 whatever the position: the first round of partials (4 MR slices) is
  // requested before the position has arrived and masked by the slice count afterwards (a partial past the live range is
  // whatever an earlier step left there: it is selected away, never used in arithmetic).
  const bool ahead = p.window <= 0 && d < hd;
  const float* pt0 = hpart + ((int64_t)seq * h_q_heads + qh) * h_n_splits * (hd + 2);
  float v[MR], ms[MR], ls[MR];
  if (ahead) {
#pragma unroll
    for (int u = 0; u < MR; u++) {
      const float* ps = pt0 + (int64_t)min(quarter + 4 * u, h_n_splits - 1) * (hd + 2);
      v[u] = ps[d]; ms[u] = ps[hd]; ls[u] = ps[hd + 1];
    }
  }
  const LiveRows lr = live_rows(p, hpos[seq]);
  const int s_first = lr.j_start / hsl, s_last = (lr.len - 1) / hsl;
  const int n_active = s_last - s_first + 1;
  if (n_active == 1) return;                       // the split kernel already wrote the final row
  const float* pt = pt0 + (int64_t)s_first * (hd + 2);
  float A = 0.0f, L = 0.0f, M = -1e30f;
  if (d < hd) {
    for (int s0 = quarter; s0 < n_active; s0 += 4 * MR) {
      if (!(ahead && s0 == quarter)) {
#pragma unroll
        for (int u = 0; u < MR; u++) {
          const float* ps = pt + (int64_t)min(s0 + 4 * u, n_active - 1) * (hd + 2);
          v[u] = ps[d]; ms[u] = ps[hd]; ls[u] = ps[hd + 1];
        }
      }
#pragma unroll
      for (int u = 0; u < MR; u++) {
        if (s0 + 4 * u < n_active && ls[u] > 0.0f) {
          const float mn = fmaxf(M, ms[u]), c0 = expf(M - mn), c1 = expf(ms[u] - mn);
          A = fmaf(v[u], c1, A * c0); L = fmaf(ls[u], c1, L * c0); M = mn;
        }
      }
    }
    qA[quarter][d] = A;
    if (d == 0) { qM[quarter] = M; qL[quarter] = L; }
  }
  __syncthreads();
  if (quarter == 0 && d < hd) {
    const float Mx = fmaxf(fmaxf(qM[0], qM[1]), fmaxf(qM[2], qM[3]));
    float At = 0.0f, Lt = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const float e = qL[k] > 0.0f ? expf(qM[k] - Mx) : 0.0f;
      At = fmaf(qA[k][d], e, At); Lt = fmaf(qL[k], e, Lt);
    }
    hout[(int64_t)seq * hout_stride + qh * hd + d] = Lt > 0.0f ? At * (1.0f / Lt) : 0.0f;
  }
}

// ---- short caches: one work-group per (split, QUERY head).  The G heads of a group each re-read the slice (from
//      L2: their work-groups are numbered so that they land on the same XCD), but no work-group loops over heads:
//      with one wave per SIMD that loop is a chain of dependent DPP/exp/LDS latencies and dominated the step.
//      Running state lives in registers; LDS is used once, for the meeting of the 8 half-waves. ----
// The leading scalar arguments are the ones the first requests need (position, the step's q | k | v row, rotary frequencies,
// grid geometry): they arrive preloaded in scalar registers (see the Makefile), so the position request leaves at once and the
// rest of the parameter block is fetched while it is on its way.  hheads = query heads | KV heads << 16, hgeo = slices | head
// width << 16.
template <int DS, typename KV_T>
__global__ __launch_bounds__(256) void attn_split_head_kernel(const int32_t* hpos, const float* hqkv, const float* htheta, const long long hqkv_stride,
                                                              const int hheads, const int hgeo, const AttnParams p)
{
  const unsigned long long tl0 = timeline_now();
  const int q_heads = hheads & 0xffff, kv_heads = hheads >> 16, n_splits = hgeo & 0xffff, hd = hgeo >> 16;
  const int G = q_heads / kv_heads;
  // linear id = item_lo + 8 * (h + G * item_hi), item = split + n_splits * kv_head: consecutive ids rotate over the XCDs
  const int L = blockIdx.x, item = (L & 7) + 8 * ((L >> 3) / G), h = (L >> 3) % G;
  if (item >= n_splits * kv_heads) return;
  const int split = item % n_splits, g = item / n_splits, seq = blockIdx.y;
  const int pos = hpos[seq];
  // the query elements and the frequencies do not depend on the position: requested behind it, before anything waits
  const int tid = threadIdx.x, hw = tid >> 5, l32 = tid & 31;
  const int qw = q_heads * hd, kw = kv_heads * hd;
  const int d0 = l32 * DS;
  const float* row = hqkv + (int64_t)seq * hqkv_stride;
  float qraw[DS], qmate = 0.0f, th[(DS + 1) / 2];
  {
    const float* qp = row + (g * G + h) * hd;
#pragma unroll
    for (int i = 0; i < DS; i++) qraw[i] = qp[min(d0 + i, hd - 1)];          // (lanes beyond the head width read its last element; the values are dropped)
    if (DS == 1) qmate = qp[min(d0 ^ 1, hd - 1)];
#pragma unroll
    for (int i = 0; i < (DS + 1) / 2; i++) th[i] = htheta ? htheta[min(d0 + 2 * i, hd - 1) >> 1] : 0.0f;
  }
  const LiveRows lr = live_rows(p, pos);
  const int len = lr.len, j_start = lr.j_start, slot = lr.slot;
  const int s_begin = max(j_start, split * p.split_len), s_end = min(len, (split + 1) * p.split_len);
  if (s_begin >= s_end) return;   // whole work-group leaves together, before any barrier
  const int s_first = j_start / p.split_len, s_last = (len - 1) / p.split_len;
  const int n_active = s_last - s_first + 1;
  timeline_put(p.timeline, 0, tl0);
  timeline_stamp(p.timeline, 1);

  KV_T* kc = reinterpret_cast<KV_T*>(p.kc) + (seq * p.seq_mul + p.seq0) * p.seq_elems + p.layer_off + (int64_t)g * p.max_ctx * hd;
  KV_T* vc = reinterpret_cast<KV_T*>(p.vc) + (seq * p.seq_mul + p.seq0) * p.seq_elems + p.layer_off + (int64_t)g * p.max_ctx * hd;

  // int8 cache: codes enter the dot products as they are; the K row scale multiplies the finished score and the V row
  // scale the softmax weight (neural/neural.cl:2639-2640, 2683-2684), so nothing is dequantised per element
  constexpr bool I8 = sizeof(KV_T) == 1;
  const float* ksc = nullptr; const float* vsc = nullptr;
  if (I8) {
    const int64_t r0 = (seq * p.seq_mul + p.seq0) * p.seq_rows + p.layer_row_off + (int64_t)g * p.max_ctx;
    ksc = p.ksc + r0; vsc = p.vsc + r0;
  }

  constexpr int PCH = 4;
  struct Chunk { float k[PCH][DS], v[PCH][DS], ks[PCH], vs[PCH]; };
  Chunk cA = {}, cB = {};
  auto load_chunk = [&](Chunk& ch, int j0) {
    if (j0 >= s_end || d0 >= hd) return;       // lanes beyond the head width keep their zeros
#pragma unroll
    for (int c = 0; c < PCH; c++) {
      const int j = min(j0 + 8 * c, s_end - 1);
      // (the slot of the row being appended may hold stale values: reduce_chunk replaces it from registers)
      load_row_vec<DS, KV_T>(kc + (int64_t)j * hd + d0, ch.k[c]);
      load_row_vec<DS, KV_T>(vc + (int64_t)j * hd + d0, ch.v[c]);
      if (I8) { ch.ks[c] = ksc[j]; ch.vs[c] = vsc[j]; }
    }
  };
  // Requests return in the order they were issued: the step's own q, k, v elements and the rotary frequencies go out first, the
  // cached rows behind them, so that the rotation (sine and cosine of an exact angle) runs while the rows are on their way
  // instead of after them.
  const bool owns_new = !p.appended && slot >= s_begin && slot < s_end;
  float kraw[DS], vraw[DS], kmate = 0.0f;
  {
    const float* kp = row + qw + g * hd; const float* vp = row + qw + kw + g * hd;
#pragma unroll
    for (int i = 0; i < DS; i++) {
      const int d = min(d0 + i, hd - 1);
      kraw[i] = owns_new ? kp[d] : 0.0f; vraw[i] = owns_new ? vp[d] : 0.0f;
    }
    if (DS == 1) kmate = owns_new ? kp[min(d0 ^ 1, hd - 1)] : 0.0f;
  }
  load_chunk(cA, s_begin + hw);
  load_chunk(cB, s_begin + hw + 8 * PCH);

  // Full-width RMSNorm of q and k (neural/neuralpretrained.pas:16511-16530) folded into this kernel: every work-group
  // sums the squares of the whole q and k rows itself (same order as the stand-alone kernel: strided per thread, wave
  // totals, (w0 + w1) + (w2 + w3)) and scales the elements it reads.
  float inv_q = 1.0f, inv_k = 1.0f;
  if (p.qn_gain) {
    __shared__ float nred[8];
    float sq = 0.0f, sk = 0.0f;
    for_strided8(row, tid, qw, 256, [&](float v, int) { sq = fmaf(v, v, sq); });
    for_strided8(row + qw, tid, kw, 256, [&](float v, int) { sk = fmaf(v, v, sk); });
    sq = wave_sum(sq); sk = wave_sum(sk);
    if ((tid & 63) == 63) { nred[tid >> 6] = sq; nred[4 + (tid >> 6)] = sk; }
    __syncthreads();
    inv_q = 1.0f / sqrtf(((nred[0] + nred[1]) + (nred[2] + nred[3])) / (float)qw + p.qk_eps);
    inv_k = 1.0f / sqrtf(((nred[4] + nred[5]) + (nred[6] + nred[7])) / (float)kw + p.qk_eps);
  }
  float rs[(DS + 1) / 2], rc[(DS + 1) / 2];
#pragma unroll
  for (int i = 0; i < (DS + 1) / 2; i++) {
    rs[i] = 0.0f; rc[i] = 1.0f;
    const int d = d0 + 2 * i;
    if (p.theta && d < hd) { const float angle = (float)pos * th[i]; sincosf(angle, &rs[i], &rc[i]); }
  }
  // raw elements (own DS, for DS = 1 also the pair's other element) -> optional RMSNorm gain -> optional rotation
  auto finish_rot = [&](const float (&raw)[DS], float mate_raw, float (&o)[DS], bool rotate, const float* gain, float inv) {
    auto elem = [&](float v, int d) { return d < hd ? (gain ? gain[d] * (v * inv) : v) : 0.0f; };
    if (DS >= 2) {
#pragma unroll
      for (int i = 0; i < DS; i += 2) {
        const int d = d0 + i;
        const float x0 = elem(raw[i], d), x1 = elem(raw[i + (DS > 1 ? 1 : 0)], d + 1);
        if (rotate) { o[i] = rc[i / 2] * x0 - rs[i / 2] * x1; o[i + (DS > 1 ? 1 : 0)] = rs[i / 2] * x0 + rc[i / 2] * x1; }
        else { o[i] = x0; o[i + (DS > 1 ? 1 : 0)] = x1; }
      }
    } else {
      const int d = d0;
      const float own = elem(raw[0], d), mate = elem(mate_raw, d ^ 1);
      if (rotate) o[0] = (d & 1) ? (rs[0] * mate + rc[0] * own) : (rc[0] * own - rs[0] * mate);
      else o[0] = own;
    }
  };
  float q[DS], knew[DS], vnew[DS], acc[DS];
  finish_rot(qraw, qmate, q, p.theta != nullptr, p.qn_gain ? p.qn_gain + (g * G + h) * hd : nullptr, inv_q);
#pragma unroll
  for (int i = 0; i < DS; i++) { acc[i] = 0.0f; knew[i] = 0.0f; vnew[i] = 0.0f; }
  // every work-group whose slice holds `pos` keeps the new row in registers; the group's first head appends it
  float knew_s = 1.0f, vnew_s = 1.0f;
  if (owns_new) {
    finish_rot(kraw, kmate, knew, p.theta != nullptr, p.kn_gain ? p.kn_gain + g * hd : nullptr, inv_k);
    finish_rot(vraw, 0.0f, vnew, false, nullptr, 1.0f);
    if constexpr (I8) {
      knew_s = quantise_row_i8<DS>(knew);
      vnew_s = quantise_row_i8<DS>(vnew);
      if (h == 0 && hw == 0) {
#pragma unroll
        for (int i = 0; i < DS; i++)
          if (d0 + i < hd) { kc[(int64_t)slot * hd + d0 + i] = (int8_t)knew[i]; vc[(int64_t)slot * hd + d0 + i] = (int8_t)vnew[i]; }
        if (l32 == 0) { p.ksc[(ksc - p.ksc) + slot] = knew_s; p.vsc[(vsc - p.vsc) + slot] = vnew_s; }
      }
    } else {
#pragma unroll
      for (int i = 0; i < DS; i++) {
        vnew[i] = kv_to_float<KV_T>(kv_from_float<KV_T>(vnew[i]));
        knew[i] = kv_to_float<KV_T>(kv_from_float<KV_T>(knew[i]));
        if (h == 0 && hw == 0 && d0 + i < hd) {
          kc[(int64_t)slot * hd + d0 + i] = kv_from_float<KV_T>(knew[i]);
          vc[(int64_t)slot * hd + d0 + i] = kv_from_float<KV_T>(vnew[i]);
        }
      }
    }
  }
  float m = -1e30f, l = 0.0f;
  timeline_stamp_after(p.timeline, 4, q[0]);
  auto reduce_chunk = [&](Chunk& ch, int j0) {
    float sc[PCH], cmax = -1e30f;
#pragma unroll
    for (int c = 0; c < PCH; c++) {
      if (owns_new && min(j0 + 8 * c, s_end - 1) == slot) {
#pragma unroll
        for (int i = 0; i < DS; i++) { ch.k[c][i] = knew[i]; ch.v[c][i] = vnew[i]; }
        if (I8) { ch.ks[c] = knew_s; ch.vs[c] = vnew_s; }
      }
      float s = 0.0f;
#pragma unroll
      for (int i = 0; i < DS; i++) s = fmaf(q[i], ch.k[c][i], s);
      s = half_wave_allsum(s) * (I8 ? ch.ks[c] * p.inv_sqrt : p.inv_sqrt);
      if (p.softcap > 0.0f) s = p.softcap * tanhf(s / p.softcap);
      sc[c] = (j0 + 8 * c < s_end) ? s : -1e30f;
      cmax = fmaxf(cmax, sc[c]);
    }
    const float mn = fmaxf(m, cmax), corr = expf(m - mn);
    float lsum = 0.0f;
#pragma unroll
    for (int i = 0; i < DS; i++) acc[i] *= corr;
#pragma unroll
    for (int c = 0; c < PCH; c++) {
      const float pj = (j0 + 8 * c < s_end) ? expf(sc[c] - mn) : 0.0f;
      lsum += pj;
      const float pv = I8 ? pj * ch.vs[c] : pj;
#pragma unroll
      for (int i = 0; i < DS; i++) acc[i] = fmaf(pv, ch.v[c][i], acc[i]);
    }
    l = l * corr + lsum; m = mn;
  };
  for (int j0 = s_begin + hw; j0 < s_end; j0 += 16 * PCH) {
    reduce_chunk(cA, j0);
    if (j0 + 16 * PCH < s_end) load_chunk(cA, j0 + 16 * PCH);
    if (j0 + 8 * PCH < s_end) {
      reduce_chunk(cB, j0 + 8 * PCH);
      if (j0 + 24 * PCH < s_end) load_chunk(cB, j0 + 24 * PCH);
    }
  }

  // ---- meeting of the 8 half-waves ----
  timeline_stamp(p.timeline, 5);
  __shared__ float sm[8], sl[8];
  __shared__ float sacc[8][32 * DS];
  if (l32 == 0) { sm[hw] = m; sl[hw] = l; }
#pragma unroll
  for (int i = 0; i < DS; i++) sacc[hw][d0 + i] = acc[i];
  __syncthreads();
  if (tid < hd) {
    const int d = tid;
    float M = -1e30f;
#pragma unroll
    for (int w = 0; w < 8; w++) M = fmaxf(M, sm[w]);
    float Ls = 0.0f, A = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; w++) {
      const float e = sl[w] > 0.0f ? expf(sm[w] - M) : 0.0f;
      Ls = fmaf(sl[w], e, Ls); A = fmaf(sacc[w][d], e, A);
    }
    const int qh = g * G + h;
    if (n_active == 1) {
      p.out[(int64_t)seq * p.out_stride + qh * hd + d] = Ls > 0.0f ? A * (1.0f / Ls) : 0.0f;
    } else {
      float* pt = p.part + (((int64_t)seq * p.q_heads + qh) * p.n_splits + split) * (hd + 2);
      if (p.merge_cnt) { part_store(pt + d, A); if (d == 0) { part_store(pt + hd, M); part_store(pt + hd + 1, Ls); } }
      else { pt[d] = A; if (d == 0) { pt[hd] = M; pt[hd + 1] = Ls; } }
    }
  }
  if (n_active > 1 && p.merge_cnt) merge_if_last(p, seq, g * G + h, 1, s_first, n_active, seq * p.kv_heads * 8 + g * G + h);
  timeline_stamp(p.timeline, 7);
}

template <typename KV_T>
static int launch_split_head(const AttnParams& p0, int n_seq, hipStream_t st)
{
  AttnParams p = p0;
  const int G = p.q_heads / p.kv_heads;
  const int items = p.n_splits * p.kv_heads;
  const dim3 grid(8 * G * ((items + 7) / 8), n_seq);
  p.timeline = timeline_next((int)(grid.x * grid.y));
  const int hheads = p.q_heads | p.kv_heads << 16, hgeo = p.n_splits | p.hd << 16;
  if (p.q_heads > 0xffff || p.kv_heads > 0x7fff || p.n_splits > 0xffff) return set_error(CAI_ERR_UNSUPPORTED, "attention: %d query heads, %d slices", p.q_heads, p.n_splits);
  const long long qs = (long long)p.qkv_stride;
  if (p.hd <= 32) hipLaunchKernelGGL((attn_split_head_kernel<1, KV_T>), grid, dim3(256), 0, st, p.pos, (const float*)p.qkv, p.theta, qs, hheads, hgeo, p);
  else if (p.hd <= 64) hipLaunchKernelGGL((attn_split_head_kernel<2, KV_T>), grid, dim3(256), 0, st, p.pos, (const float*)p.qkv, p.theta, qs, hheads, hgeo, p);
  else if (p.hd <= 128) hipLaunchKernelGGL((attn_split_head_kernel<4, KV_T>), grid, dim3(256), 0, st, p.pos, (const float*)p.qkv, p.theta, qs, hheads, hgeo, p);
  else return set_error(CAI_ERR_UNSUPPORTED, "attention: head_dim %d > 128", p.hd);
  return CAI_OK;
}

template <typename KV_T, int NPF>
static void launch_group_t(const AttnParams& p0, const dim3 grid, size_t lds, int hc, hipStream_t st)
{
  AttnParams p = p0;
  p.timeline = timeline_next((int)(grid.x * grid.y));
  switch (hc) {
#define CAI_GROUP_ARGS p.pos, (const float*)p.qkv, p.theta, (long long)p.qkv_stride, p.q_heads | p.kv_heads << 16, p.n_splits | p.hd << 16, p.split_len, p
    case 1: hipLaunchKernelGGL((attn_group_kernel<1, KV_T, NPF>), grid, dim3(256), lds, st, CAI_GROUP_ARGS); break;
    case 2: hipLaunchKernelGGL((attn_group_kernel<2, KV_T, NPF>), grid, dim3(256), lds, st, CAI_GROUP_ARGS); break;
    case 3: hipLaunchKernelGGL((attn_group_kernel<3, KV_T, NPF>), grid, dim3(256), lds, st, CAI_GROUP_ARGS); break;
    case 4: hipLaunchKernelGGL((attn_group_kernel<4, KV_T, NPF>), grid, dim3(256), lds, st, CAI_GROUP_ARGS); break;
    case 5: hipLaunchKernelGGL((attn_group_kernel<5, KV_T, NPF>), grid, dim3(256), lds, st, CAI_GROUP_ARGS); break;
    case 6: hipLaunchKernelGGL((attn_group_kernel<6, KV_T, NPF>), grid, dim3(256), lds, st, CAI_GROUP_ARGS); break;
    case 7: hipLaunchKernelGGL((attn_group_kernel<7, KV_T, NPF>), grid, dim3(256), lds, st, CAI_GROUP_ARGS); break;
    default: hipLaunchKernelGGL((attn_group_kernel<8, KV_T, NPF>), grid, dim3(256), lds, st, CAI_GROUP_ARGS); break;
#undef CAI_GROUP_ARGS
  }
}

template <typename KV_T>
static int launch_group(const AttnParams& p, int n_seq, hipStream_t st)
{
  const int G = p.q_heads / p.kv_heads;
  constexpr int hc_max = 8;    // query heads held in registers per pass
  const int n_chunks = (G + hc_max - 1) / hc_max, hc = (G + n_chunks - 1) / n_chunks;
  const dim3 grid(p.n_splits * p.kv_heads, n_seq);
  const size_t lds = (size_t)(G * 128 + G * p.split_len + n_chunks * p.split_len * (hc > 4 ? 8 : 4) + 4 * hc * 128 + 2 * G) * sizeof(float);
  if (lds > 64 * 1024) return set_error(CAI_ERR_UNSUPPORTED, "attention: %d query heads per KV head need %zu bytes of LDS", G, lds);
  // Several work-groups per CU: a shallow load ring frees registers for more resident waves (5 instead of 3 per SIMD),
  // which hides the phase changes of one work-group behind the streaming of the others.  A grid of about one work-group
  // per CU has nothing to overlap with and keeps the deep ring.
  if ((int)(grid.x * grid.y) >= 3 * ctx().n_cu) launch_group_t<KV_T, 2>(p, grid, lds, hc, st);
  else launch_group_t<KV_T, (sizeof(KV_T) == 4 ? 4 : 8)>(p, grid, lds, hc, st);
  return CAI_OK;
}

// Whether the grouped launch of this cache takes the matrix-core kernel (CAIHIP_ATTN_GROUP_MFMA=0 keeps the VALU form).
static bool group_takes_mfma(const AttnParams& p, int dtype)
{
  static const bool on = []() { const char* e = getenv("CAIHIP_ATTN_GROUP_MFMA"); return !(e && e[0] == '0'); }();
  return on && (dtype == CAI_KV_F16 || dtype == CAI_KV_I8) && p.hd == 128 && p.q_heads / p.kv_heads <= 16 && p.split_len <= 256;
}
template <typename KV_T>
static int launch_group_mfma(const AttnParams& p0, int n_seq, hipStream_t st)
{
  AttnParams p = p0;
  const dim3 grid(p.n_splits * p.kv_heads, n_seq);
  p.timeline = timeline_next((int)(grid.x * grid.y));
  if (p.q_heads > 0xffff || p.kv_heads > 0x7fff || p.n_splits > 0xffff) return set_error(CAI_ERR_UNSUPPORTED, "attention: %d query heads, %d slices", p.q_heads, p.n_splits);
  const int hheads = p.q_heads | p.kv_heads << 16, hgeo = p.n_splits | p.hd << 16;
#define CAI_GM_LAUNCH(TPWv, NWv) do { \
    static bool attr_done = false;      /* up to 80 KB of dynamic LDS */ \
    if (!attr_done) { CAI_HIP(hipFuncSetAttribute((const void*)attn_group_mfma_kernel<TPWv, NWv, KV_T>, hipFuncAttributeMaxDynamicSharedMemorySize, gm_lds_bytes(TPWv, NWv))); attr_done = true; } \
    hipLaunchKernelGGL((attn_group_mfma_kernel<TPWv, NWv, KV_T>), grid, dim3(64 * NWv), gm_lds_bytes(TPWv, NWv), st, p.pos, (const float*)p.qkv, p.theta, (long long)p.qkv_stride, hheads, hgeo, p.split_len, p); } while (0)
  // slices of up to 128 rows: four waves; longer ones: eight (32B shape at 8.2k rows, slices of 256: 177.5 tok/s with four waves
  // of four tiles, 180.8 with eight waves of two at batch 1; 693.7 against 698.0 at batch 8)
  if (p.split_len <= 128) CAI_GM_LAUNCH(2, 4);
  else CAI_GM_LAUNCH(2, 8);
#undef CAI_GM_LAUNCH
  return CAI_OK;
}

// Prompt ingestion: rotate the K rows of n_tok tokens at their positions and write K,V into sequence `seq`.
template <typename KV_T>
__device__ __forceinline__ void kv_append_row(const AttnParams& p)
{
  const int b = blockIdx.x;
  const float* row = p.qkv + (int64_t)b * p.qkv_stride;
  const int pos = p.pos[b], slot = live_rows(p, pos).slot;
  const int hd = p.hd, qw = p.q_heads * hd, kw = p.kv_heads * hd;
  KV_T* kc = reinterpret_cast<KV_T*>(p.kc) + (int64_t)p.seq0 * p.seq_elems + p.layer_off;
  KV_T* vc = reinterpret_cast<KV_T*>(p.vc) + (int64_t)p.seq0 * p.seq_elems + p.layer_off;
  for (int i = threadIdx.x; i < (kw >> 1); i += 256) {
    const int e = 2 * i, g = e / hd, d = e % hd;
    float x0 = row[qw + e], x1 = row[qw + e + 1];
    if (p.theta) {
      const float angle = (float)pos * p.theta[d >> 1];
      float sn, cs; sincosf(angle, &sn, &cs);
      const float y0 = cs * x0 - sn * x1, y1 = sn * x0 + cs * x1;
      x0 = y0; x1 = y1;
    }
    KV_T* dst = kc + ((int64_t)g * p.max_ctx + slot) * hd + d;
    dst[0] = kv_from_float<KV_T>(x0); dst[1] = kv_from_float<KV_T>(x1);
  }
  for (int i = threadIdx.x; i < kw; i += 256) {
    const int g = i / hd, d = i % hd;
    vc[((int64_t)g * p.max_ctx + slot) * hd + d] = kv_from_float<KV_T>(row[qw + kw + i]);
  }
}
template <typename KV_T>
__global__ __launch_bounds__(256) void kv_append_rows_kernel(const AttnParams p) { kv_append_row<KV_T>(p); }

// The same for an int8 cache: one half-wave per (token, KV head, K|V) row, quantised with the decode step's rule.
template <int DS>
__global__ __launch_bounds__(256) void kv_append_rows_i8_kernel(const AttnParams p)
{
  const int b = blockIdx.x, hw = threadIdx.x >> 5, l32 = threadIdx.x & 31;
  const float* row = p.qkv + (int64_t)b * p.qkv_stride;
  const int pos = p.pos[b], slot = live_rows(p, pos).slot;
  const int hd = p.hd, qw = p.q_heads * hd, kw = p.kv_heads * hd;
  const int d0 = l32 * DS;
  for (int item = hw; item < 2 * p.kv_heads; item += 8) {      // uniform per half-wave; both halves of a wave loop alike
    const int g = item >> 1, is_v = item & 1;
    const float* src = row + qw + (is_v ? kw : 0) + g * hd;
    float v[DS];
    if (DS >= 2) {
#pragma unroll
      for (int i = 0; i < DS; i += 2) {
        const int d = d0 + i;
        float x0 = d < hd ? src[d] : 0.0f, x1 = d + 1 < hd ? src[d + 1] : 0.0f;
        if (p.theta && !is_v && d < hd) {
          float sn, cs; sincosf((float)pos * p.theta[d >> 1], &sn, &cs);
          const float y0 = cs * x0 - sn * x1, y1 = sn * x0 + cs * x1;
          x0 = y0; x1 = y1;
        }
        v[i] = x0; v[i + (DS > 1 ? 1 : 0)] = x1;
      }
    } else {
      const int d = d0;
      const float own = d < hd ? src[d] : 0.0f, mate = (d ^ 1) < hd ? src[d ^ 1] : 0.0f;
      v[0] = own;
      if (p.theta && !is_v && d < hd) {
        float sn, cs; sincosf((float)pos * p.theta[d >> 1], &sn, &cs);
        v[0] = (d & 1) ? (sn * mate + cs * own) : (cs * own - sn * mate);
      }
    }
    const float scale = quantise_row_i8<DS>(v);
    const int64_t srow = (int64_t)p.seq0 * p.seq_rows + p.layer_row_off + (int64_t)g * p.max_ctx + slot;
    int8_t* dst = reinterpret_cast<int8_t*>(is_v ? p.vc : p.kc) + (int64_t)p.seq0 * p.seq_elems + p.layer_off + ((int64_t)g * p.max_ctx + slot) * hd;
#pragma unroll
    for (int i = 0; i < DS; i++) if (d0 + i < hd) dst[d0 + i] = (int8_t)v[i];
    if (l32 == 0) (is_v ? p.vsc : p.ksc)[srow] = scale;
  }
}

// ------------------------------------------------------------------------------------------
// Prompt ingestion on the matrix cores: every prompt token attends over the cached rows up to its own position.
// Work-group = (KV head, four query heads of its group, 32 consecutive tokens); wave w takes head h0 + w.  K and V
// tiles of 32 cached rows are staged in LDS (V transposed) and shared by the four waves.  Per tile and wave:
//   S^T[row][token] = K . q^T   on v_mfma_f32_32x32x8_f16: the result lane holds ONE token column, so the running
//                               maximum, the normaliser and the rescaling of the output are per-lane scalars, and the
//                               result registers of k-step s are exactly the B operand of step s of the next product;
//   O^T[dim][token] += V^T . P^T   with P split hi + lo into two f16 (22 bits), like q; a float cache is split too.
// Same arithmetic as the decode kernels up to the order of the sums (tests: < 1e-4 of token-at-a-time ingestion).
// ------------------------------------------------------------------------------------------
typedef float pf16_t __attribute__((ext_vector_type(16)));

struct PromptParams {
  const float* qkv; int64_t qkv_stride;      // rows [Q | K | V], K and V already appended to the cache
  _Float16* qhi; _Float16* qlo;              // [token][q_heads * 128] rotated q, hi + lo
  const void* kc; const void* vc;            // this sequence's layer plane: [kv_head][max_ctx][128]
  const float* ksc; const float* vsc;        // int8 cache: row scales of the same plane, [kv_head][max_ctx]
  int q_heads, kv_heads, max_ctx, n_tok, window;
  float softcap, inv_sqrt;
  const float* theta; const int32_t* pos;
  float* out; int64_t out_stride;
  float* part;                               // [token][q_head][K split][128 + 2]: unnormalised sums, maximum, normaliser
};

constexpr int PA_KT_MIN = 2;     // K tiles (of 32 cached rows) a split takes at least
constexpr int PA_KS_MAX = 8;     // splits of a token tile's K range at most
// K tiles a token tile walks and the number of work-groups (blockIdx.z) they are cut over: long ranges are split so that a
// short prompt (few token tiles, a causal triangle of work) still fills the chip; the merge kernel adds the pieces.
__device__ __forceinline__ void prompt_k_range(const PromptParams& p, int t0, int n_ks, int& jt0, int& jt1, int& splits)
{
  const int pos_first = p.pos[t0], pos_last = p.pos[min(t0 + 31, p.n_tok - 1)];
  const int j_lo = (p.window > 0 && pos_first + 1 > p.window) ? pos_first + 1 - p.window : 0;
  jt0 = j_lo >> 5; jt1 = pos_last >> 5;
  splits = max(1, min(n_ks, (jt1 - jt0 + 1) / PA_KT_MIN));
}

// rotated q (neural/neural.cl:1517-1542) as two f16 planes
__device__ __forceinline__ void prompt_q_row(const PromptParams& p)
{
  const int t = blockIdx.x, qw = p.q_heads * 128;
  const float* row = p.qkv + (int64_t)t * p.qkv_stride;
  const int pos = p.pos[t];
  for (int e = threadIdx.x; e < (qw >> 1); e += 256) {
    const int d = (2 * e) & 127;
    float x0 = row[2 * e], x1 = row[2 * e + 1];
    if (p.theta) {
      float sn, cs; sincosf((float)pos * p.theta[d >> 1], &sn, &cs);
      const float y0 = cs * x0 - sn * x1, y1 = sn * x0 + cs * x1;
      x0 = y0; x1 = y1;
    }
    _Float16 h0, h1, l0, l1;
    split_f16(x0, h0, l0); split_f16(x1, h1, l1);
    p.qhi[(int64_t)t * qw + 2 * e] = h0; p.qhi[(int64_t)t * qw + 2 * e + 1] = h1;
    p.qlo[(int64_t)t * qw + 2 * e] = l0; p.qlo[(int64_t)t * qw + 2 * e + 1] = l1;
  }
}
__global__ __launch_bounds__(256) void prompt_q_kernel(const PromptParams p) { prompt_q_row(p); }
// one launch per chunk for both: the token's K and V rows into the cache, its rotated q into the planes
template <typename KV_T>
__global__ __launch_bounds__(256) void prompt_rows_kernel(const AttnParams p, const PromptParams pp) { kv_append_row<KV_T>(p); prompt_q_row(pp); }

constexpr int PA_LDK = 136;    // halfs per staged K row (128 + pad: rows stay 16-byte aligned for the 8-half operand reads)
constexpr int PA_LDV = 36;     // halfs per staged V^T row (32 cached rows + pad)

template <typename KV_T>
__global__ __launch_bounds__(256) void attn_prompt_kernel(const PromptParams p)
{
  constexpr bool I8P = sizeof(KV_T) == 1;         // int8 rows are dequantised (code * row scale) while they are staged
  constexpr bool F32 = sizeof(KV_T) != 2;         // ... and, like a float cache, split hi + lo
  constexpr int NP = F32 ? 2 : 1;                 // planes of K and V
  __shared__ __align__(16) _Float16 sK[NP][32 * PA_LDK];
  __shared__ __align__(16) _Float16 sV[NP][128 * PA_LDV];
  const int G = p.q_heads / p.kv_heads, quads = (G + 3) >> 2;
  const int g = blockIdx.y / quads, h0 = (blockIdx.y % quads) * 4;
  const int t0 = blockIdx.x * 32;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 31, kg = lane >> 5;
  const int hq = h0 + wave;                       // head within the group
  const bool head_on = hq < G;
  const int head = g * G + (head_on ? hq : 0);
  const int tok = t0 + n;
  const bool tok_on = tok < p.n_tok;
  const int pos_n = tok_on ? p.pos[tok] : -1;
  const int jstart_n = (p.window > 0 && pos_n + 1 > p.window) ? pos_n + 1 - p.window : 0;
  // the tile's range of cached rows (tokens are consecutive positions of one sequence) and this work-group's share of it
  int jt_first, jt_last, splits;
  prompt_k_range(p, t0, (int)gridDim.z, jt_first, jt_last, splits);
  const int ks = blockIdx.z;
  if (ks >= splits) return;                       // (uniform: the whole work-group leaves before any barrier)
  {
    const int per = (jt_last - jt_first + 1 + splits - 1) / splits;
    const int a = jt_first + ks * per;
    jt_last = min(jt_last, a + per - 1); jt_first = a;
  }
  const KV_T* kc = reinterpret_cast<const KV_T*>(p.kc) + (int64_t)g * p.max_ctx * 128;
  const KV_T* vc = reinterpret_cast<const KV_T*>(p.vc) + (int64_t)g * p.max_ctx * 128;

  // this lane's q fragments: token n, dims 16 s + 8 kg .. + 7 of the wave's head
  ph8_t qh[8], ql[8];
  {
    const int64_t qo = (int64_t)min(tok, p.n_tok - 1) * (p.q_heads * 128) + head * 128 + 8 * kg;
#pragma unroll
    for (int s = 0; s < 8; s++) {
      qh[s] = *reinterpret_cast<const ph8_t*>(p.qhi + qo + 16 * s);
      ql[s] = *reinterpret_cast<const ph8_t*>(p.qlo + qo + 16 * s);
    }
  }
  pf16_t O[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int v = 0; v < 16; v++) O[dt][v] = 0.0f;
  float m_run = -1e30f, l_run = 0.0f;

  const int srow = tid >> 3, sdim = (tid & 7) * 16;         // staging: 16 consecutive elements of one cached row
  // The rows of the NEXT tile are requested before the products of the current one and converted into LDS after them: the
  // memory round trip runs behind the matrix-core work instead of in front of it.  Requests are unconditional (rows past the
  // live range are clamped and masked below).
  struct RawTile { uint4 k[sizeof(KV_T) == 4 ? 4 : 2], v[sizeof(KV_T) == 4 ? 4 : 2]; float ks, vs; };   // (int8: one uint4 each is used)
  auto fetch = [&](int jt, RawTile& r) {
    const int j = min(jt * 32 + srow, p.max_ctx - 1);
    if (I8P) {
      r.k[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const int8_t*>(kc) + (int64_t)j * 128 + sdim);
      r.v[0] = *reinterpret_cast<const uint4*>(reinterpret_cast<const int8_t*>(vc) + (int64_t)j * 128 + sdim);
      r.ks = p.ksc[(int64_t)g * p.max_ctx + j]; r.vs = p.vsc[(int64_t)g * p.max_ctx + j];
    } else if (sizeof(KV_T) == 4) {
#pragma unroll
      for (int c4 = 0; c4 < 4; c4++) {
        r.k[c4] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(kc) + (int64_t)j * 128 + sdim + 4 * c4);
        r.v[c4] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(vc) + (int64_t)j * 128 + sdim + 4 * c4);
      }
    } else {
#pragma unroll
      for (int c8 = 0; c8 < 2; c8++) {
        r.k[c8] = *reinterpret_cast<const uint4*>(reinterpret_cast<const __half*>(kc) + (int64_t)j * 128 + sdim + 8 * c8);
        r.v[c8] = *reinterpret_cast<const uint4*>(reinterpret_cast<const __half*>(vc) + (int64_t)j * 128 + sdim + 8 * c8);
      }
    }
  };
  RawTile raw;
  fetch(jt_first, raw);
  for (int jt = jt_first; jt <= jt_last; jt++) {
    __syncthreads();                                        // the previous tile has been consumed
    {
      float kv[16], vv[16];
      if (I8P) {
        const uint4 a = raw.k[0], b = raw.v[0];
        const float ks = raw.ks, vs = raw.vs;
        const int aw[4] = {(int)a.x, (int)a.y, (int)a.z, (int)a.w}, bw[4] = {(int)b.x, (int)b.y, (int)b.z, (int)b.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
          kv[4 * i] = (float)((aw[i] << 24) >> 24) * ks; kv[4 * i + 1] = (float)((aw[i] << 16) >> 24) * ks;
          kv[4 * i + 2] = (float)((aw[i] << 8) >> 24) * ks; kv[4 * i + 3] = (float)(aw[i] >> 24) * ks;
          vv[4 * i] = (float)((bw[i] << 24) >> 24) * vs; vv[4 * i + 1] = (float)((bw[i] << 16) >> 24) * vs;
          vv[4 * i + 2] = (float)((bw[i] << 8) >> 24) * vs; vv[4 * i + 3] = (float)(bw[i] >> 24) * vs;
        }
      } else if (sizeof(KV_T) == 4) {
#pragma unroll
        for (int c4 = 0; c4 < 4; c4++) {
          const uint4 a = raw.k[c4], b = raw.v[c4];
          kv[4 * c4] = __builtin_bit_cast(float, a.x); kv[4 * c4 + 1] = __builtin_bit_cast(float, a.y); kv[4 * c4 + 2] = __builtin_bit_cast(float, a.z); kv[4 * c4 + 3] = __builtin_bit_cast(float, a.w);
          vv[4 * c4] = __builtin_bit_cast(float, b.x); vv[4 * c4 + 1] = __builtin_bit_cast(float, b.y); vv[4 * c4 + 2] = __builtin_bit_cast(float, b.z); vv[4 * c4 + 3] = __builtin_bit_cast(float, b.w);
        }
      }
      if constexpr (sizeof(KV_T) == 2) {                  // a half cache goes in as it is
#pragma unroll
        for (int c8 = 0; c8 < 2; c8++) {
          const uint4 a = raw.k[c8], b = raw.v[c8];
          *reinterpret_cast<uint2*>(&sK[0][srow * PA_LDK + sdim + 8 * c8]) = make_uint2(a.x, a.y);
          *reinterpret_cast<uint2*>(&sK[0][srow * PA_LDK + sdim + 8 * c8 + 4]) = make_uint2(a.z, a.w);
          const uint32_t bw[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
          for (int i = 0; i < 4; i++) {
            sV[0][(sdim + 8 * c8 + 2 * i) * PA_LDV + srow] = __builtin_bit_cast(_Float16, (unsigned short)(bw[i] & 0xffffu));
            sV[0][(sdim + 8 * c8 + 2 * i + 1) * PA_LDV + srow] = __builtin_bit_cast(_Float16, (unsigned short)(bw[i] >> 16));
          }
        }
      } else {
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {                    // K rows stay row-major: 8-byte stores
        ph4_t kh, kl;
#pragma unroll
        for (int i = 0; i < 4; i++) { _Float16 a, b; split_f16(kv[4 * i4 + i], a, b); kh[i] = a; kl[i] = b; }
        *reinterpret_cast<ph4_t*>(&sK[0][srow * PA_LDK + sdim + 4 * i4]) = kh;
        if (F32) *reinterpret_cast<ph4_t*>(&sK[NP - 1][srow * PA_LDK + sdim + 4 * i4]) = kl;
      }
#pragma unroll
      for (int i = 0; i < 16; i++) {                      // V goes in transposed
        _Float16 vh, vl; split_f16(vv[i], vh, vl);
        sV[0][(sdim + i) * PA_LDV + srow] = vh;
        if (F32) sV[NP - 1][(sdim + i) * PA_LDV + srow] = vl;
      }
      }
    }
    fetch(jt + 1, raw);                                     // in flight during the products below
    __syncthreads();
    if (!head_on) continue;                                 // (an idle wave still stages and meets the barriers)

    // ---- S^T = K . q^T ----
    pf16_t C;
#pragma unroll
    for (int v = 0; v < 16; v++) C[v] = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; s++) {
      const ph8_t a = *reinterpret_cast<const ph8_t*>(&sK[0][n * PA_LDK + 16 * s + 8 * kg]);
      C = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qh[s], C, 0, 0, 0);
      C = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, ql[s], C, 0, 0, 0);
      if (F32) {
        const ph8_t al = *reinterpret_cast<const ph8_t*>(&sK[NP - 1][n * PA_LDK + 16 * s + 8 * kg]);
        C = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, qh[s], C, 0, 0, 0);
      }
    }
    // ---- this token's column: mask, running maximum, weights ----
    float tmax = -1e30f;
    bool ok[16];
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int krow = jt * 32 + 8 * (v >> 2) + 4 * kg + (v & 3);
      float sc = C[v] * p.inv_sqrt;
      if (p.softcap > 0.0f) sc = p.softcap * tanhf(sc / p.softcap);
      ok[v] = krow <= pos_n && krow >= jstart_n;
      C[v] = sc;
      if (ok[v]) tmax = fmaxf(tmax, sc);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax), corr = expf(m_run - m_new);
    float psum = 0.0f;
#pragma unroll
    for (int v = 0; v < 16; v++) { C[v] = ok[v] ? expf(C[v] - m_new) : 0.0f; psum += C[v]; }
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * corr + psum; m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(corr != 1.0f)) {      // (after the first tiles a new maximum is rare: the whole wave skips the rescaling)
#pragma unroll
      for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) O[dt][v] *= corr;
    }
    // ---- O^T += V^T . P^T ----
    // The score registers 8 s2 .. 8 s2 + 7 of a lane are cached rows 16 s2 + 4 kg + (0..3) and 16 s2 + 8 + 4 kg + (0..3): taken as
    // the eight k of a 16-deep step, with the value operand read as the same two groups of four rows (the order of the
    // rows inside a step is free as long as both operands agree).
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++) {
      ph8_t ph, pl;
#pragma unroll
      for (int i = 0; i < 8; i++) { _Float16 hv, lv; split_f16(C[8 * s2 + i], hv, lv); ph[i] = hv; pl[i] = lv; }
#pragma unroll
      for (int dt = 0; dt < 4; dt++) {
        const ph4_t a0 = *reinterpret_cast<const ph4_t*>(&sV[0][(32 * dt + n) * PA_LDV + 16 * s2 + 4 * kg]);
        const ph4_t a1 = *reinterpret_cast<const ph4_t*>(&sV[0][(32 * dt + n) * PA_LDV + 16 * s2 + 8 + 4 * kg]);
        const ph8_t a = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, ph, O[dt], 0, 0, 0);
        O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pl, O[dt], 0, 0, 0);
        if (F32) {
          const ph4_t b0 = *reinterpret_cast<const ph4_t*>(&sV[NP - 1][(32 * dt + n) * PA_LDV + 16 * s2 + 4 * kg]);
          const ph4_t b1 = *reinterpret_cast<const ph4_t*>(&sV[NP - 1][(32 * dt + n) * PA_LDV + 16 * s2 + 8 + 4 * kg]);
          const ph8_t al = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
          O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, ph, O[dt], 0, 0, 0);
        }
      }
    }
  }
  if (!head_on || !tok_on) return;
  if (splits > 1) {        // this piece's unnormalised sums, maximum and normaliser; prompt_merge_kernel adds the pieces
    float* pt = p.part + (((int64_t)tok * p.q_heads + head) * gridDim.z + ks) * 130;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        float* q4 = pt + 32 * dt + 8 * g4 + 4 * kg;       // (130-float records: 8-byte aligned only)
        q4[0] = O[dt][4 * g4]; q4[1] = O[dt][4 * g4 + 1]; q4[2] = O[dt][4 * g4 + 2]; q4[3] = O[dt][4 * g4 + 3];
      }
    if (kg == 0) { pt[128] = m_run; pt[129] = l_run; }
    return;
  }
  const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
  float* dst = p.out + (int64_t)tok * p.out_stride + head * 128;
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int g4 = 0; g4 < 4; g4++)
      *reinterpret_cast<float4*>(dst + 32 * dt + 8 * g4 + 4 * kg) =
          make_float4(O[dt][4 * g4] * inv, O[dt][4 * g4 + 1] * inv, O[dt][4 * g4 + 2] * inv, O[dt][4 * g4 + 3] * inv);
}

// out[token][head] = sum of the K splits of a token tile, folded with a running maximum in split order (a tile walked by one
// work-group was written by it and is left alone)
__global__ __launch_bounds__(512) void prompt_merge_kernel(const PromptParams p, int n_ks)
{
  const int tok = blockIdx.x, head = blockIdx.y * 4 + (threadIdx.x >> 7), d = threadIdx.x & 127;   // four heads per work-group
  int jt0, jt1, splits;
  prompt_k_range(p, (tok >> 5) << 5, n_ks, jt0, jt1, splits);
  if (splits <= 1 || head >= p.q_heads) return;
  const float* pt = p.part + (((int64_t)tok * p.q_heads + head) * n_ks) * 130;
  float M = -1e30f, L = 0.0f, A = 0.0f;
  float ms[PA_KS_MAX], ls[PA_KS_MAX], as[PA_KS_MAX];                     // all requests first (a split past the count repeats the last one; not used)
#pragma unroll
  for (int s = 0; s < PA_KS_MAX; s++) { const int sc = min(s, splits - 1); ms[s] = pt[sc * 130 + 128]; ls[s] = pt[sc * 130 + 129]; as[s] = pt[sc * 130 + d]; }
#pragma unroll
  for (int s = 0; s < PA_KS_MAX; s++) {
    if (s < splits && ls[s] > 0.0f) {
      const float mn = fmaxf(M, ms[s]), c0 = expf(M - mn), c1 = expf(ms[s] - mn);
      A = A * c0 + as[s] * c1; L = L * c0 + ls[s] * c1; M = mn;
    }
  }
  p.out[(int64_t)tok * p.out_stride + head * 128 + d] = L > 0.0f ? A * (1.0f / L) : 0.0f;
}

// Whether n prompt rows of this cache go to the matrix-core prompt kernel (it needs no per-slice partial results).
bool attn_prompt_is_flash(const cai_kv_s* kv, int n)
{
  static const int flash_on = []() { const char* e = getenv("CAIHIP_PROMPT_FLASH"); return e ? atoi(e) : 1; }();
  return flash_on && kv->head_dim == 128 && kv->evict_cap == 0 && n >= 8;
}

int launch_attn_step(cai_kv_s* kv, int layer, float* qkv, int64_t qkv_stride, int n_seq, int q_heads, int window,
                     float softcap, const float* theta, const int32_t* pos_dev, float* out, int64_t out_stride, int seq0,
                     int prompt_rows, float* prompt_part, const float* qn_gain, const float* kn_gain, float qk_eps)
{
  Context& c = ctx();
  if (layer < 0 || layer >= kv->n_layers) return set_error(CAI_ERR_INVALID, "attention: layer %d of %d", layer, kv->n_layers);
  if (n_seq < 1 || seq0 < 0 || seq0 + (prompt_rows ? 1 : n_seq) > kv->n_seq) return set_error(CAI_ERR_INVALID, "attention: %d sequences, cache holds %d", n_seq, kv->n_seq);
  if (q_heads % kv->kv_heads) return set_error(CAI_ERR_INVALID, "attention: %d query heads not a multiple of %d KV heads", q_heads, kv->kv_heads);
  if (q_heads > kv->part_q_heads) return set_error(CAI_ERR_INVALID, "attention: %d query heads exceed the cache's scratch (%d)", q_heads, kv->part_q_heads);
  AttnParams p{};
  p.qkv = qkv; p.qkv_stride = qkv_stride; p.kc = kv->k; p.vc = kv->v;
  p.seq_elems = kv->seq_elems(); p.layer_off = (int64_t)layer * kv->layer_elems();
  p.q_heads = q_heads; p.kv_heads = kv->kv_heads; p.hd = kv->head_dim; p.max_ctx = kv->max_ctx;
  p.window = window; p.softcap = softcap; p.inv_sqrt = kv->score_mul / sqrtf((float)kv->head_dim);
  p.theta = theta; p.pos = pos_dev;
  if (kv->geo_rows > 0) {   // the caller chose a length bucket: it must cover the rows the host knows to be in use
    int needed = 0;
    for (int s0 = 0; s0 < (prompt_rows ? 1 : n_seq); s0++) needed = std::max(needed, kv->len_at(seq0 + s0, layer) + (prompt_rows ? n_seq : 1));
    if (needed > kv->geo_rows) return set_error(CAI_ERR_STATE, "attention: launch geometry covers %d rows, %d are in use", kv->geo_rows, needed);
  }
  kv_geometry(kv, kv->geo_rows, &p.split_len, &p.n_splits);
  p.part = prompt_rows ? prompt_part : kv->part; p.out = out; p.out_stride = out_stride; p.seq0 = seq0;
  p.seq_mul = prompt_rows ? 0 : 1; p.appended = prompt_rows ? 1 : 0;
  p.evict_sinks = kv->evict_sinks; p.evict_cap = kv->evict_cap;
  p.ksc = kv->ks; p.vsc = kv->vs; p.seq_rows = kv->seq_rows(); p.layer_row_off = (int64_t)layer * kv->layer_rows();
  int rc;
  const int group_min = c.n_cu;   // smallest grid that fills the chip with one work-group per (slice, KV head)
  // (a cache short enough to be ONE slice may be up to 2048 rows long: the grouped kernel's per-slice score arrays in LDS are
  // sized for ordinary slices, the per-head kernel keeps its state in registers)
  const bool grouped = (kv->head_dim & 7) == 0 && p.split_len <= 256 && n_seq * kv->kv_heads * p.n_splits >= group_min;
  // The per-head kernel merges its slices itself (one work-group per head does a head's merge).  A prompt has more rows in
  // flight than the counters cover, and in the per-KV-head kernel the last arriver would fold a whole group of heads over
  // many slices alone (32B shape, 33 slices x 5 heads: 37.7 us against 30.7 us with the merge launch): those keep the launch.
  p.merge_cnt = (prompt_rows || grouped) ? nullptr : kv->merge_cnt;
  if (qn_gain) {
    // q and k norms over the whole rows: the per-head decode kernel applies them while it reads its operands; the
    // other kernels find the rows normalised in place
    const int qw = q_heads * kv->head_dim, kw = kv->kv_heads * kv->head_dim;
    if (!prompt_rows && !grouped) { p.qn_gain = qn_gain; p.kn_gain = kn_gain; p.qk_eps = qk_eps; }
    else if ((rc = launch_rmsnorm_pair(qkv, qn_gain, qw, kn_gain, kw, n_seq, qk_eps, qkv_stride))) return rc;
  }
  // prompts over a 128-wide cache: matrix-core kernel, 32 tokens x 4 heads per work-group
  const bool flash = prompt_rows == 1 && attn_prompt_is_flash(kv, n_seq);
  const bool rows_fused = flash && kv->dtype != CAI_KV_I8;     // the append and the q planes share a launch (below)
  if (prompt_rows && kv->dtype == CAI_KV_I8) {
    if (p.hd <= 32) hipLaunchKernelGGL(kv_append_rows_i8_kernel<1>, dim3(n_seq), dim3(256), 0, c.stream, p);
    else if (p.hd <= 64) hipLaunchKernelGGL(kv_append_rows_i8_kernel<2>, dim3(n_seq), dim3(256), 0, c.stream, p);
    else hipLaunchKernelGGL(kv_append_rows_i8_kernel<4>, dim3(n_seq), dim3(256), 0, c.stream, p);
  } else if (prompt_rows && !rows_fused) {
    if (kv->dtype == CAI_KV_F16) hipLaunchKernelGGL(kv_append_rows_kernel<__half>, dim3(n_seq), dim3(256), 0, c.stream, p);
    else hipLaunchKernelGGL(kv_append_rows_kernel<float>, dim3(n_seq), dim3(256), 0, c.stream, p);
  }
  if (flash) {
    const size_t need = (size_t)n_seq * q_heads * 128;
    if (need > kv->pq_cap) {
      CAI_HIP(hipStreamSynchronize(c.stream));
      if (kv->pq_hi) (void)hipFree(kv->pq_hi);
      if (kv->pq_lo) (void)hipFree(kv->pq_lo);
      kv->pq_hi = kv->pq_lo = nullptr; kv->pq_cap = 0;
      CAI_HIP(hipMalloc(&kv->pq_hi, need * 2));
      CAI_HIP(hipMalloc(&kv->pq_lo, need * 2));
      kv->pq_cap = need;
    }
    PromptParams pp{};
    pp.qkv = qkv; pp.qkv_stride = qkv_stride; pp.qhi = (_Float16*)kv->pq_hi; pp.qlo = (_Float16*)kv->pq_lo;
    const size_t plane = ((size_t)seq0 * kv->seq_elems() + (size_t)layer * kv->layer_elems()) * kv->elem();
    pp.kc = (const char*)kv->k + plane; pp.vc = (const char*)kv->v + plane;
    if (kv->dtype == CAI_KV_I8) {
      const size_t rows0 = (size_t)seq0 * kv->seq_rows() + (size_t)layer * kv->layer_rows();
      pp.ksc = kv->ks + rows0; pp.vsc = kv->vs + rows0;
    }
    pp.q_heads = q_heads; pp.kv_heads = kv->kv_heads; pp.max_ctx = kv->max_ctx; pp.n_tok = n_seq; pp.window = window;
    pp.softcap = softcap; pp.inv_sqrt = p.inv_sqrt; pp.theta = theta; pp.pos = pos_dev; pp.out = out; pp.out_stride = out_stride;
    const int G = q_heads / kv->kv_heads;
    const int wgs = ((n_seq + 31) / 32) * kv->kv_heads * ((G + 3) / 4);
    // K splits per token tile: as many as keep the launch at one work-group per CU (a tile with few K tiles takes fewer).
    // Measured on 511 tokens of the 7B shape (128 work-groups unsplit): 67 us -> 38.7 + 11.2 us (merge) with two splits,
    // 50.8 + 11.6 with three; on 512-token chunks of the 32B shape (256 work-groups) splitting loses (365 -> 373 + 16 us).
    const int n_ks = std::max(1, std::min(PA_KS_MAX, c.n_cu / wgs));
    if (n_ks > 1) {
      const size_t pneed = (size_t)n_seq * q_heads * n_ks * 130;
      if (pneed > kv->pq_part_cap) {
        CAI_HIP(hipStreamSynchronize(c.stream));
        if (kv->pq_part) (void)hipFree(kv->pq_part);
        kv->pq_part = nullptr; kv->pq_part_cap = 0;
        CAI_HIP(hipMalloc((void**)&kv->pq_part, pneed * 4));
        kv->pq_part_cap = pneed;
      }
    }
    pp.part = kv->pq_part;
    if (!rows_fused) hipLaunchKernelGGL(prompt_q_kernel, dim3(n_seq), dim3(256), 0, c.stream, pp);
    else if (kv->dtype == CAI_KV_F16) hipLaunchKernelGGL(prompt_rows_kernel<__half>, dim3(n_seq), dim3(256), 0, c.stream, p, pp);
    else hipLaunchKernelGGL(prompt_rows_kernel<float>, dim3(n_seq), dim3(256), 0, c.stream, p, pp);
    const dim3 grid((n_seq + 31) / 32, kv->kv_heads * ((G + 3) / 4), n_ks);
    if (kv->dtype == CAI_KV_F16) hipLaunchKernelGGL(attn_prompt_kernel<__half>, grid, dim3(256), 0, c.stream, pp);
    else if (kv->dtype == CAI_KV_I8) hipLaunchKernelGGL(attn_prompt_kernel<int8_t>, grid, dim3(256), 0, c.stream, pp);
    else hipLaunchKernelGGL(attn_prompt_kernel<float>, grid, dim3(256), 0, c.stream, pp);
    if (n_ks > 1) hipLaunchKernelGGL(prompt_merge_kernel, dim3(n_seq, (q_heads + 3) / 4), dim3(512), 0, c.stream, pp, n_ks);
    return CAI_OK;
  }
  // one work-group per (slice, KV head) serving the whole group of query heads, or one per (slice, query head)
  // (the first fetches K and V once but has G times fewer work-groups: it needs a grid that fills the chip by itself)
  if (grouped && group_takes_mfma(p, kv->dtype))
    rc = kv->dtype == CAI_KV_I8 ? launch_group_mfma<int8_t>(p, n_seq, c.stream) : launch_group_mfma<__half>(p, n_seq, c.stream);
  else if (grouped)
    rc = kv->dtype == CAI_KV_I8 ? launch_group<int8_t>(p, n_seq, c.stream) : kv->dtype == CAI_KV_F16 ? launch_group<__half>(p, n_seq, c.stream) : launch_group<float>(p, n_seq, c.stream);
  else
    rc = kv->dtype == CAI_KV_I8 ? launch_split_head<int8_t>(p, n_seq, c.stream) : kv->dtype == CAI_KV_F16 ? launch_split_head<__half>(p, n_seq, c.stream) : launch_split_head<float>(p, n_seq, c.stream);
  if (rc) return rc;
  if (p.n_splits > 1 && !p.merge_cnt)
  {
    if (p.n_splits > 96)
      hipLaunchKernelGGL(attn_merge_kernel<32>, dim3(q_heads, n_seq), dim3(512), 0, c.stream, p.pos, (const float*)p.part, p.out, (long long)p.out_stride,
                         p.q_heads | p.kv_heads << 16, p.n_splits | p.hd << 16, p.split_len, p);
    else
      hipLaunchKernelGGL(attn_merge_kernel<12>, dim3(q_heads, n_seq), dim3(512), 0, c.stream, p.pos, (const float*)p.part, p.out, (long long)p.out_stride,
                         p.q_heads | p.kv_heads << 16, p.n_splits | p.hd << 16, p.split_len, p);
  }
  return CAI_OK;
}

// ------------------------------------------------------------------------------------------
// cache lifetime
// ------------------------------------------------------------------------------------------
int kv_bucket_rows(const cai_kv_s* kv, int needed_rows)
{
  if (kv->evict_cap > 0) return 0;                       // a rolling cache is short by construction: its own geometry
  int rows = 1024;
  while (rows < needed_rows && rows < kv->max_ctx) rows *= 2;
  return rows >= kv->max_ctx ? 0 : rows;
}

void kv_geometry(const cai_kv_s* kv, int rows, int* split_len, int* n_splits)
{
  if (rows <= 0 || rows > kv->max_ctx) rows = kv->max_ctx;
  // few, fat slices: every extra slice costs the merging work-group another device-coherent load round,
  // while one CU sustains only ~20 GB/s, so a slice should stay under ~100 KB
  constexpr int sl_max = 256;
  int sl = (rows + 15) / 16; sl = (sl + 31) / 32 * 32; if (sl < 32) sl = 32; if (sl > sl_max) sl = sl_max;
  // From 8192 rows on the grouped kernel (K and V fetched once for all query heads of a KV head) is the fast one, but it needs
  // about one work-group per CU: with few KV heads the slices are halved until slices x KV heads fill the chip.  7B shape, 4 KV
  // heads, 7000 rows: 256-row slices take the per-head kernel at 31.8 us per launch, 128-row slices the grouped one at 23.3
  // (445 -> 494 tok/s); at 4096 rows both forms take the same time and the longer slices stay.
  if (rows >= 8192 && (kv->head_dim & 7) == 0)
    while (sl > 64 && kv->kv_heads * ((rows + sl - 1) / sl) < ctx().n_cu) sl /= 2;
  // a head's whole K (or V) plane of at most 64 KB is one slice: a single work-group streams it in a few microseconds and
  // the merge launch disappears (small models at short contexts are bound by launches, not by bytes)
  constexpr int single_bytes = 65536;
  if ((int64_t)rows * kv->head_dim * (kv->dtype == CAI_KV_F16 ? 2 : kv->dtype == CAI_KV_I8 ? 1 : 4) <= single_bytes) sl = (rows + 31) / 32 * 32;
  *split_len = sl; *n_splits = (rows + sl - 1) / sl;
}

int kv_alloc(cai_kv_s* kv, int n_seq, int n_layers, int kv_heads, int head_dim, int max_ctx, int dtype)
{
  if (n_seq < 1 || n_layers < 1 || kv_heads < 1 || head_dim < 2 || (head_dim & 1) || (head_dim > 64 && (head_dim & 3)) || head_dim > 128 || max_ctx < 1)
    return set_error(CAI_ERR_INVALID, "kv cache: bad geometry seq=%d layers=%d kv_heads=%d head_dim=%d max_ctx=%d", n_seq, n_layers, kv_heads, head_dim, max_ctx);
  if (dtype != CAI_KV_F32 && dtype != CAI_KV_F16 && dtype != CAI_KV_I8) return set_error(CAI_ERR_INVALID, "kv cache: dtype %d", dtype);
  kv->n_seq = n_seq; kv->n_layers = n_layers; kv->kv_heads = kv_heads; kv->head_dim = head_dim; kv->max_ctx = max_ctx; kv->dtype = dtype;
  kv->len.assign((size_t)n_seq * n_layers, 0);
  kv->geo_rows = 0;
  kv_geometry(kv, 0, &kv->split_len, &kv->n_splits);
  kv->n_splits_alloc = kv->n_splits;
  for (int rows = 1024; rows < max_ctx; rows *= 2) { int sl, ns; kv_geometry(kv, rows, &sl, &ns); kv->n_splits_alloc = std::max(kv->n_splits_alloc, ns); }
  const size_t bytes = (size_t)kv->seq_elems() * n_seq * kv->elem();
  // (the kernels index slices generically; the bound keeps the per-row scratch of prompts and windows - one partial result per
  // slice and query head - within reason: 131072 rows are 512 slices)
  if (kv->n_splits > 512) return set_error(CAI_ERR_UNSUPPORTED, "kv cache: max_ctx %d needs %d slices of %d rows (limit 512: 131072 rows)", max_ctx, kv->n_splits, kv->split_len);
  CAI_HIP(hipMalloc(&kv->k, bytes));
  CAI_HIP(hipMalloc(&kv->v, bytes));
  CAI_HIP(hipMemsetAsync(kv->k, 0, bytes, ctx().stream));
  CAI_HIP(hipMemsetAsync(kv->v, 0, bytes, ctx().stream));
  if (dtype == CAI_KV_I8) {
    const size_t sb = (size_t)kv->seq_rows() * n_seq * sizeof(float);
    CAI_HIP(hipMalloc(&kv->ks, sb));
    CAI_HIP(hipMalloc(&kv->vs, sb));
    CAI_HIP(hipMemsetAsync(kv->ks, 0, sb, ctx().stream));
    CAI_HIP(hipMemsetAsync(kv->vs, 0, sb, ctx().stream));
  }
  kv->part_q_heads = kv_heads * 8;
  CAI_HIP(hipMalloc(&kv->part, (size_t)n_seq * kv->part_q_heads * kv->n_splits_alloc * (head_dim + 2) * sizeof(float)));
  CAI_HIP(hipMalloc(&kv->d_len, sizeof(int32_t) * n_seq));
  CAI_HIP(hipMalloc((void**)&kv->merge_cnt, sizeof(unsigned) * n_seq * kv->part_q_heads));
  CAI_HIP(hipMemsetAsync(kv->merge_cnt, 0, sizeof(unsigned) * n_seq * kv->part_q_heads, ctx().stream));
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  return CAI_OK;
}

void kv_free(cai_kv_s* kv)
{
  if (kv->k) (void)hipFree(kv->k);
  if (kv->v) (void)hipFree(kv->v);
  if (kv->ks) (void)hipFree(kv->ks);
  if (kv->vs) (void)hipFree(kv->vs);
  kv->ks = kv->vs = nullptr;
  if (kv->pq_hi) (void)hipFree(kv->pq_hi);
  if (kv->pq_lo) (void)hipFree(kv->pq_lo);
  if (kv->pq_part) (void)hipFree(kv->pq_part);
  kv->pq_hi = kv->pq_lo = nullptr; kv->pq_cap = 0; kv->pq_part = nullptr; kv->pq_part_cap = 0;
  if (kv->part) (void)hipFree(kv->part);
  if (kv->d_len) (void)hipFree(kv->d_len);
  if (kv->merge_cnt) (void)hipFree(kv->merge_cnt);
  kv->merge_cnt = nullptr;
  kv->k = kv->v = nullptr; kv->part = nullptr; kv->d_len = nullptr;
}

// Deep copy of the live rows of one sequence (TNNetDecoderSessionSnapshot, neural/neuraldecode.pas:1089-1142).
int kv_snapshot(cai_kv_s* kv, int seq, cai_kv_snap_s** out)
{
  cai_kv_snap_s* s = new cai_kv_snap_s();
  auto drop = [&](int code) { cai_kv_snap_destroy(s); return code; };   // every error path releases what the snapshot holds so far
  s->n_layers = kv->n_layers; s->kv_heads = kv->kv_heads; s->head_dim = kv->head_dim; s->dtype = kv->dtype;
  s->evict_sinks = kv->evict_sinks; s->evict_cap = kv->evict_cap;
  s->len.resize(kv->n_layers);
  int rows = 0;
  for (int l = 0; l < kv->n_layers; l++) { s->len[l] = kv->len_at(seq, l); rows = std::max(rows, kv->live(s->len[l])); }
  s->rows = rows;
  if (rows > 0) {
    const size_t bytes = (size_t)kv->n_layers * kv->kv_heads * rows * kv->head_dim * kv->elem();
    if (hipMalloc(&s->k, bytes) != hipSuccess || hipMalloc(&s->v, bytes) != hipSuccess)
      return (void)hipGetLastError(), drop(set_error(CAI_ERR_NOMEM, "kv snapshot: out of device memory (%zu bytes)", 2 * bytes));
    const size_t row_b = (size_t)kv->head_dim * kv->elem();
    for (int which = 0; which < 2; which++) {
      const char* src = (const char*)(which ? kv->v : kv->k) + (size_t)seq * kv->seq_elems() * kv->elem();
      char* dst = (char*)(which ? s->v : s->k);
      // [layer*kv_heads] planes of max_ctx rows -> planes of `rows` rows
      const hipError_t e = hipMemcpy2DAsync(dst, (size_t)rows * row_b, src, (size_t)kv->max_ctx * row_b, (size_t)rows * row_b,
                                            (size_t)kv->n_layers * kv->kv_heads, hipMemcpyDeviceToDevice, ctx().stream);
      if (e != hipSuccess) return drop(hip_fail(e, "kv snapshot copy", __FILE__, __LINE__));
    }
    if (kv->dtype == CAI_KV_I8) {     // the row scales travel with the codes
      const size_t sb = (size_t)kv->n_layers * kv->kv_heads * rows * sizeof(float);
      if (hipMalloc(&s->ks, sb) != hipSuccess || hipMalloc(&s->vs, sb) != hipSuccess)
        return (void)hipGetLastError(), drop(set_error(CAI_ERR_NOMEM, "kv snapshot: out of device memory (%zu bytes)", 2 * sb));
      for (int which = 0; which < 2; which++) {
        const hipError_t e = hipMemcpy2DAsync(which ? s->vs : s->ks, (size_t)rows * 4, (which ? kv->vs : kv->ks) + (size_t)seq * kv->seq_rows(), (size_t)kv->max_ctx * 4,
                                              (size_t)rows * 4, (size_t)kv->n_layers * kv->kv_heads, hipMemcpyDeviceToDevice, ctx().stream);
        if (e != hipSuccess) return drop(hip_fail(e, "kv snapshot copy", __FILE__, __LINE__));
      }
    }
    { const hipError_t e = hipStreamSynchronize(ctx().stream); if (e != hipSuccess) return drop(hip_fail(e, "kv snapshot sync", __FILE__, __LINE__)); }
  }
  *out = s;
  return CAI_OK;
}

int kv_restore(cai_kv_s* kv, int seq, const cai_kv_snap_s* s)
{
  if (s->n_layers != kv->n_layers || s->kv_heads != kv->kv_heads || s->head_dim != kv->head_dim)
    return set_error(CAI_ERR_INVALID, "kv restore: snapshot geometry differs from the cache");
  if (s->dtype != kv->dtype) return set_error(CAI_ERR_INVALID, "kv restore: snapshot element type differs from the cache (mode must match)");
  if (s->evict_sinks != kv->evict_sinks || s->evict_cap != kv->evict_cap)
    return set_error(CAI_ERR_INVALID, "kv restore: snapshot was taken under eviction (%d sinks, cap %d), the cache runs (%d, %d)", s->evict_sinks, s->evict_cap, kv->evict_sinks, kv->evict_cap);
  if (s->rows > kv->max_ctx) return set_error(CAI_ERR_INVALID, "kv restore: snapshot holds %d rows, cache %d", s->rows, kv->max_ctx);
  if (s->rows > 0) {
    const size_t row_b = (size_t)kv->head_dim * kv->elem();
    for (int which = 0; which < 2; which++) {
      char* dst = (char*)(which ? kv->v : kv->k) + (size_t)seq * kv->seq_elems() * kv->elem();
      const char* src = (const char*)(which ? s->v : s->k);
      CAI_HIP(hipMemcpy2DAsync(dst, (size_t)kv->max_ctx * row_b, src, (size_t)s->rows * row_b, (size_t)s->rows * row_b,
                               (size_t)kv->n_layers * kv->kv_heads, hipMemcpyDeviceToDevice, ctx().stream));
    }
    if (kv->dtype == CAI_KV_I8)
      for (int which = 0; which < 2; which++)
        CAI_HIP(hipMemcpy2DAsync((which ? kv->vs : kv->ks) + (size_t)seq * kv->seq_rows(), (size_t)kv->max_ctx * 4, which ? s->vs : s->ks, (size_t)s->rows * 4,
                                 (size_t)s->rows * 4, (size_t)kv->n_layers * kv->kv_heads, hipMemcpyDeviceToDevice, ctx().stream));
    CAI_HIP(hipStreamSynchronize(ctx().stream));
  }
  for (int l = 0; l < kv->n_layers; l++) kv->len_at(seq, l) = s->len[l];
  return CAI_OK;
}

// Sequence dst becomes a copy of sequence src (the cache-forking step of a beam search: every survivor continues from its
// parent's rows, neural/neuraldecode.pas:1436-1449): the live rows of every (layer, KV head) plane move device to device, on
// the library's stream, without a snapshot in between.
int kv_fork(cai_kv_s* kv, int src, int dst)
{
  if (src == dst) return CAI_OK;
  int rows = 0;
  for (int l = 0; l < kv->n_layers; l++) rows = std::max(rows, kv->live(kv->len_at(src, l)));
  if (rows > 0) {
    const size_t row_b = (size_t)kv->head_dim * kv->elem(), seq_b = (size_t)kv->seq_elems() * kv->elem();
    for (int which = 0; which < 2; which++) {
      char* base = (char*)(which ? kv->v : kv->k);
      CAI_HIP(hipMemcpy2DAsync(base + dst * seq_b, (size_t)kv->max_ctx * row_b, base + src * seq_b, (size_t)kv->max_ctx * row_b, (size_t)rows * row_b,
                               (size_t)kv->n_layers * kv->kv_heads, hipMemcpyDeviceToDevice, ctx().stream));
    }
    if (kv->dtype == CAI_KV_I8)
      for (int which = 0; which < 2; which++) {
        float* base = which ? kv->vs : kv->ks;
        CAI_HIP(hipMemcpy2DAsync(base + (size_t)dst * kv->seq_rows(), (size_t)kv->max_ctx * 4, base + (size_t)src * kv->seq_rows(), (size_t)kv->max_ctx * 4,
                                 (size_t)rows * 4, (size_t)kv->n_layers * kv->kv_heads, hipMemcpyDeviceToDevice, ctx().stream));
      }
  }
  for (int l = 0; l < kv->n_layers; l++) kv->len_at(dst, l) = kv->len_at(src, l);
  return CAI_OK;
}

}  // namespace cai

// ------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------
using namespace cai;

extern "C" int cai_kv_create(int n_layers, int kv_heads, int head_dim, int max_ctx, int kv_dtype, cai_kv_t* out)
{
  CAI_ENTER();
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
  CAI_ENTER();
  if (!kv) return CAI_OK;
  (void)hipStreamSynchronize(ctx().stream);
  kv_free(kv); delete kv;
  return CAI_OK;
}

extern "C" int cai_kv_reset(cai_kv_t kv)
{
  CAI_ENTER();
  CAI_REQUIRE(kv, "cai_kv_reset: null cache");
  std::fill(kv->len.begin(), kv->len.end(), 0);
  return CAI_OK;
}

extern "C" int cai_kv_truncate(cai_kv_t kv, int n)
{
  CAI_ENTER();
  CAI_REQUIRE(kv, "cai_kv_truncate: null cache");
  CAI_REQUIRE(n >= 0, "cai_kv_truncate: negative length %d", n);
  for (int l : kv->len)
    if (l > n && kv->evict_cap > 0 && l > kv->evict_cap) return set_error(CAI_ERR_STATE, "cai_kv_truncate: %d tokens streamed under eviction, the rows before %d are gone", l, l - (kv->evict_cap - kv->evict_sinks));
  for (auto& l : kv->len) if (l > n) l = n;
  return CAI_OK;
}

// Sink + recent-window eviction (TNNetStreamingDecoder.EnableEviction / DisableEviction, neural/neuraldecode.pas:5722-5735).
int cai::kv_set_eviction(cai_kv_s* kv, int sinks, int recent)
{
  const int cap = sinks + recent;
  if (sinks < 0 || recent < 0 || (cap > 0 && recent < 1)) return set_error(CAI_ERR_INVALID, "eviction: %d sink tokens, recent window %d", sinks, recent);
  if (cap > kv->max_ctx) return set_error(CAI_ERR_INVALID, "eviction: %d sinks + %d recent exceed the cache's %d rows", sinks, recent, kv->max_ctx);
  // rows sit at slot = position until the stream passes the cap, so the policy may change freely before that
  const int limit = std::min(kv->evict_cap > 0 ? kv->evict_cap : kv->max_ctx, cap > 0 ? cap : kv->max_ctx);
  for (int n : kv->len)
    if (n > limit) return set_error(CAI_ERR_STATE, "eviction: a sequence already holds %d tokens, past the %d the change allows", n, limit);
  kv->evict_sinks = cap > 0 ? sinks : 0; kv->evict_cap = cap;
  return CAI_OK;
}

extern "C" int cai_kv_set_eviction(cai_kv_t kv, int sink_tokens, int recent_window)
{
  CAI_ENTER();
  CAI_REQUIRE(kv, "cai_kv_set_eviction: null cache");
  return kv_set_eviction(kv, sink_tokens, recent_window);
}

extern "C" int cai_kv_rows(cai_kv_t kv, int layer, int* rows_out)
{
  CAI_ENTER();
  CAI_REQUIRE(kv && rows_out, "cai_kv_rows: null argument");
  CAI_REQUIRE(layer >= 0 && layer < kv->n_layers, "cai_kv_rows: layer %d of %d", layer, kv->n_layers);
  *rows_out = kv->live(kv->len_at(0, layer));
  return CAI_OK;
}

extern "C" int cai_kv_len(cai_kv_t kv, int layer, int* len_out)
{
  CAI_ENTER();
  CAI_REQUIRE(kv && len_out, "cai_kv_len: null argument");
  CAI_REQUIRE(layer >= 0 && layer < kv->n_layers, "cai_kv_len: layer %d of %d", layer, kv->n_layers);
  *len_out = kv->len_at(0, layer);
  return CAI_OK;
}

extern "C" int cai_kv_snapshot(cai_kv_t kv, cai_kv_snap_t* out)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(kv && out, "cai_kv_snapshot: null argument");
  return kv_snapshot(kv, 0, out);
}

extern "C" int cai_kv_restore(cai_kv_t kv, cai_kv_snap_t snap)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(kv && snap, "cai_kv_restore: null argument");
  return kv_restore(kv, 0, snap);
}

extern "C" int cai_kv_snap_destroy(cai_kv_snap_t s)
{
  CAI_ENTER();
  if (!s) return CAI_OK;
  if (s->k) (void)hipFree(s->k);
  if (s->v) (void)hipFree(s->v);
  if (s->ks) (void)hipFree(s->ks);
  if (s->vs) (void)hipFree(s->vs);
  delete s;
  return CAI_OK;
}

// one layer of sequence 0 <-> packed host rows; dir 0 = device to host
static int kv_layer_copy(cai_kv_s* kv, int layer, int len, void* k, void* v, float* ks, float* vs, int to_device)
{
  if (len == 0) return CAI_OK;
  const size_t row_b = (size_t)kv->head_dim * kv->elem();
  const hipMemcpyKind kind = to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost;
  auto copy2d = [&](char* dev, char* host, size_t unit) -> hipError_t {
    return to_device ? hipMemcpy2DAsync(dev, (size_t)kv->max_ctx * unit, host, (size_t)len * unit, (size_t)len * unit, (size_t)kv->kv_heads, kind, ctx().stream)
                     : hipMemcpy2DAsync(host, (size_t)len * unit, dev, (size_t)kv->max_ctx * unit, (size_t)len * unit, (size_t)kv->kv_heads, kind, ctx().stream);
  };
  CAI_HIP(copy2d((char*)kv->k + (size_t)layer * kv->layer_elems() * kv->elem(), (char*)k, row_b));
  CAI_HIP(copy2d((char*)kv->v + (size_t)layer * kv->layer_elems() * kv->elem(), (char*)v, row_b));
  if (kv->dtype == CAI_KV_I8) {
    CAI_HIP(copy2d((char*)(kv->ks + (size_t)layer * kv->layer_rows()), (char*)ks, 4));
    CAI_HIP(copy2d((char*)(kv->vs + (size_t)layer * kv->layer_rows()), (char*)vs, 4));
  }
  CAI_HIP(hipStreamSynchronize(ctx().stream));
  return CAI_OK;
}

extern "C" int cai_kv_export_layer(cai_kv_t kv, int layer, void* k, void* v, float* k_scales, float* v_scales)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(kv && k && v, "cai_kv_export_layer: null argument");
  CAI_REQUIRE(layer >= 0 && layer < kv->n_layers, "cai_kv_export_layer: layer %d of %d", layer, kv->n_layers);
  CAI_REQUIRE(kv->dtype != CAI_KV_I8 || (k_scales && v_scales), "cai_kv_export_layer: an int8 cache needs the scale outputs");
  return kv_layer_copy(kv, layer, kv->live(kv->len_at(0, layer)), k, v, k_scales, v_scales, 0);
}

extern "C" int cai_kv_import_layer(cai_kv_t kv, int layer, int len, const void* k, const void* v, const float* k_scales, const float* v_scales)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(kv && (len == 0 || (k && v)), "cai_kv_import_layer: null argument");
  CAI_REQUIRE(layer >= 0 && layer < kv->n_layers, "cai_kv_import_layer: layer %d of %d", layer, kv->n_layers);
  CAI_REQUIRE(len >= 0 && len <= kv->max_ctx && (kv->evict_cap == 0 || len <= kv->evict_cap), "cai_kv_import_layer: %d rows, cache holds %d", len, kv->evict_cap ? kv->evict_cap : kv->max_ctx);
  CAI_REQUIRE(kv->dtype != CAI_KV_I8 || len == 0 || (k_scales && v_scales), "cai_kv_import_layer: an int8 cache needs the row scales");
  const int rc = kv_layer_copy(kv, layer, len, const_cast<void*>(k), const_cast<void*>(v), const_cast<float*>(k_scales), const_cast<float*>(v_scales), 1);
  if (rc) return rc;
  kv->len_at(0, layer) = len;
  return CAI_OK;
}

extern "C" int cai_attn_decode(cai_kv_t kv, int layer, const float* qkv, int q_heads, int window, float softcap,
                               float* out, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(kv && qkv && out, "cai_attn_decode: null argument");
  CAI_REQUIRE(layer >= 0 && layer < kv->n_layers, "cai_attn_decode: layer %d of %d", layer, kv->n_layers);
  CAI_REQUIRE(q_heads > 0 && q_heads % kv->kv_heads == 0, "cai_attn_decode: %d query heads vs %d KV heads", q_heads, kv->kv_heads);
  Context& c = ctx();
  const int len = kv->len_at(0, layer);
  if (len >= kv->max_ctx && kv->evict_cap == 0) return set_error(CAI_ERR_STATE, "cai_attn_decode: cache full (%d rows)", kv->max_ctx);
  const int hd = kv->head_dim;
  const size_t in_b = (size_t)(q_heads + 2 * kv->kv_heads) * hd * sizeof(float), out_b = (size_t)q_heads * hd * sizeof(float);
  // the kernel rotates/append from a mutable row: always work on a private device copy
  int rc = ensure_stage(&c.stage_in, &c.stage_in_cap, in_b); if (rc) return rc;
  CAI_HIP(hipMemcpyAsync(c.stage_in, qkv, in_b, (flags & CAI_X_DEVICE) ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, c.stream));
  float* d_out = out;
  if (!(flags & CAI_Y_DEVICE)) { rc = ensure_stage(&c.stage_out, &c.stage_out_cap, out_b); if (rc) return rc; d_out = (float*)c.stage_out; }
  c.h_small[0] = len;
  CAI_HIP(hipMemcpyAsync(kv->d_len, c.h_small, sizeof(int32_t), hipMemcpyHostToDevice, c.stream));
  kv->geo_rows = kv_bucket_rows(kv, len + 1);
  rc = launch_attn_step(kv, layer, (float*)c.stage_in, 0, 1, q_heads, window, softcap, nullptr, kv->d_len, d_out, 0, 0, 0, nullptr);
  if (rc) return rc;
  if (!(flags & CAI_Y_DEVICE)) CAI_HIP(hipMemcpyAsync(out, d_out, out_b, hipMemcpyDeviceToHost, c.stream));
  CAI_HIP(hipStreamSynchronize(c.stream));
  kv->len_at(0, layer) = len + 1;
  return CAI_OK;
}
