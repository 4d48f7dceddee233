// Distribution pipeline ahead of the samplers, on the device, so that a sampled (non-greedy) decode does not read
// the vocabulary-sized logits row back (TChatEngine.GenerateFromIds, neural/neuralchatengine.pas:1374-1396, 1495-1501):
//   softmax -> history penalty in the probability domain (neural/neuralvolume.pas:5335-5376)
//           -> temperature in the probability domain (neural/neuraldecode.pas:4710-4754)
//           -> the m most probable tokens in descending order: the prefix every sampler of the reference draws from
//              (TNNetSamplerBase.SelectTopCandidates / SortTokenArray, neural/neuralvolume.pas:5171-5196; the nucleus
//              sampler starts from a 256-wide prefix itself, 4548-4562).
// The draw stays with the host and its own random generator: it gets m (token, probability) pairs instead of the row.
//
// One work-group of 1024 lanes walks the row (it sits in L2: 608 KB for a 152k vocabulary) a handful of times; the
// m-th largest probability is found exactly by a three-level radix histogram over the float bit patterns (12+12+8
// bits), ties at the threshold are taken in token order, and the survivors are rank-sorted in LDS.
#include "cai_internal.hpp"

namespace cai {

constexpr int SMP_T = 1024;
constexpr int SMP_MAX_M = 1024;

__device__ __forceinline__ float smp_block_max(float v, float* red)
{
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < SMP_T / 64; w++) r = fmaxf(r, red[w]);
  return r;
}

__device__ __forceinline__ float smp_block_sum(float v, float* red)
{
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = 0.0f;
#pragma unroll
  for (int w = 0; w < SMP_T / 64; w++) r += red[w];
  return r;
}

// exclusive prefix sum over the work-group in thread order; *total gets the sum
__device__ __forceinline__ int smp_block_excl_scan(int v, int* red, int* total)
{
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int inc = v;
  for (int o = 1; o < 64; o <<= 1) { const int t = __shfl_up(inc, o, 64); if (lane >= o) inc += t; }
  __syncthreads();
  if (lane == 63) red[w] = inc;
  __syncthreads();
  int before = 0, all = 0;
#pragma unroll
  for (int i = 0; i < SMP_T / 64; i++) { const int t = red[i]; if (i < w) before += t; all += t; }
  *total = all;
  return before + inc - v;
}

struct SampleParams {
  const float* logits; int n;
  const int32_t* hist_ids; const int32_t* hist_counts; int n_hist;
  float repetition, frequency, presence, temperature;
  int m;
  float* probs;           // n floats of scratch
  int32_t* tok_out; float* p_out;
};

__global__ __launch_bounds__(SMP_T) void candidates_kernel(const SampleParams p)
{
  __shared__ float redf[SMP_T / 64];
  __shared__ int redi[SMP_T / 64];
  __shared__ int hist[4096];
  __shared__ int sel[2];                  // chosen bin, candidates still needed inside it
  __shared__ int n_gt;
  __shared__ float cp[SMP_MAX_M];
  __shared__ int32_t ct[SMP_MAX_M];
  const int tid = threadIdx.x, n = p.n;
  float* pr = p.probs;

  // ---- softmax (stable; the same clamps as the host row softmax) ----
  float mx = -3.0e38f;
  // (every pass over the row requests eight values per thread and turn before it uses the first: see for_strided8)
  for_strided8(p.logits, tid, n, SMP_T, [&](float v, int) { mx = fmaxf(mx, v); });
  mx = smp_block_max(mx, redf);
  float sum = 0.0f;
  for_strided8(p.logits, tid, n, SMP_T, [&](float v, int i) {
    const float a = fminf(fmaxf(v - mx, -4000.0f), 4000.0f);
    const float e = expf(a);
    pr[i] = e; sum += e;
  });
  sum = smp_block_sum(sum, redf);
  if (sum > 0.0f) { const float inv = 1.0f / sum; for_strided8(pr, tid, n, SMP_T, [&](float v, int i) { pr[i] = v * inv; }); }
  __syncthreads();

  // ---- history penalty: p^r, * exp(-(f*count + presence)) on the distinct context tokens, renormalise ----
  if ((p.repetition != 1.0f || p.frequency != 0.0f || p.presence != 0.0f) && p.n_hist > 0) {
    int changed = 0;
    for (int k = tid; k < p.n_hist; k += SMP_T) {
      const int t = p.hist_ids[k];
      if (t < 0 || t >= n) continue;
      float v = pr[t];
      if (p.repetition != 1.0f && v > 0.0f) v = powf(v, p.repetition);
      if (p.frequency != 0.0f || p.presence != 0.0f) v *= expf(-(p.frequency * (float)p.hist_counts[k] + p.presence));
      pr[t] = v; changed = 1;
    }
    changed = __syncthreads_or(changed);
    if (changed) {
      float tot = 0.0f;
      for_strided8(pr, tid, n, SMP_T, [&](float v, int) { tot += v; });
      tot = smp_block_sum(tot, redf);
      if (tot > 0.0f) for_strided8(pr, tid, n, SMP_T, [&](float v, int i) { pr[i] = v / tot; });
      __syncthreads();
    }
  }

  // ---- temperature: exp(ln(max(p, 1e-30)) / T - ln(max p) / T), renormalise ----
  if (p.temperature != 1.0f) {
    const float T = fmaxf(p.temperature, 1e-6f);
    float pm = 0.0f;
    for_strided8(pr, tid, n, SMP_T, [&](float v, int) { pm = fmaxf(pm, v); });
    pm = smp_block_max(pm, redf);
    if (pm > 0.0f) {
      const float lm = logf(fmaxf(pm, 1e-30f)), inv_t = 1.0f / T;
      float s2 = 0.0f;
      for_strided8(pr, tid, n, SMP_T, [&](float q, int i) {
        const float v = expf(logf(fmaxf(q, 1e-30f)) * inv_t - lm * inv_t);
        pr[i] = v; s2 += v;
      });
      s2 = smp_block_sum(s2, redf);
      if (s2 <= 0.0f) s2 = 1.0f;
      const float inv = 1.0f / s2;
      for_strided8(pr, tid, n, SMP_T, [&](float v, int i) { pr[i] = v * inv; });
    }
    __syncthreads();
  }

  // ---- the m-th largest probability, exactly: probabilities are >= 0, so their bit patterns order like the values ----
  const int m = min(p.m, n);
  uint32_t prefix = 0, prefix_mask = 0;
  int need = m;                                  // candidates still to be taken at or below the current prefix
  const int shifts[3] = {20, 8, 0};
  const uint32_t widths[3] = {0xFFFu, 0xFFFu, 0xFFu};
  for (int lvl = 0; lvl < 3; lvl++) {
    for (int b = tid; b < 4096; b += SMP_T) hist[b] = 0;
    __syncthreads();
    for_strided8(pr, tid, n, SMP_T, [&](float v, int) {
      const uint32_t u = __float_as_uint(v);
      if ((u & prefix_mask) == prefix) atomicAdd(&hist[(u >> shifts[lvl]) & widths[lvl]], 1);
    });
    __syncthreads();
    // thread t owns the four bins 4095-4t .. 4092-4t (top bins first), so a forward scan counts what lies above
    const int b0 = 4095 - 4 * tid;
    const int own = hist[b0] + hist[b0 - 1] + hist[b0 - 2] + hist[b0 - 3];
    int total;
    const int above = smp_block_excl_scan(own, redi, &total);
    if (above < need && need <= above + own) {   // exactly one thread: the crossing lies in its bins
      int acc = above;
      for (int k = 0; k < 4; k++) {
        const int c = hist[b0 - k];
        if (need <= acc + c) { sel[0] = b0 - k; sel[1] = need - acc; break; }
        acc += c;
      }
    }
    __syncthreads();
    prefix |= (uint32_t)sel[0] << shifts[lvl]; prefix_mask |= widths[lvl] << shifts[lvl];
    need = sel[1];
    __syncthreads();
  }
  const uint32_t thr = prefix;                   // bit pattern of the m-th largest value; `need` of its copies are taken

  // ---- survivors: everything above the threshold (any order), then `need` of the equal ones in token order ----
  if (tid == 0) n_gt = 0;
  __syncthreads();
  for_strided8(pr, tid, n, SMP_T, [&](float v, int i) {
    if (__float_as_uint(v) > thr) { const int s = atomicAdd(&n_gt, 1); cp[s] = v; ct[s] = i; }
  });
  __syncthreads();
  const int base = n_gt;                         // = m - need
  {
    const int chunk = (n + SMP_T - 1) / SMP_T, i0 = tid * chunk, i1 = min(n, i0 + chunk);
    int ties = 0;
    if (i0 < i1) for_strided8(pr + i0, 0, i1 - i0, 1, [&](float v, int) { ties += __float_as_uint(v) == thr; });
    int total;
    int rank = smp_block_excl_scan(ties, redi, &total);
    if (i0 < i1 && ties > 0 && rank < need)
      for_strided8(pr + i0, 0, i1 - i0, 1, [&](float v, int i) {
        if (rank < need && __float_as_uint(v) == thr) { cp[base + rank] = v; ct[base + rank] = i0 + i; rank++; }
      });
  }
  __syncthreads();

  // ---- rank sort: descending probability, equal ones by token ----
  if (tid < m) {
    const float v = cp[tid]; const int t = ct[tid];
    int rank = 0;
    for (int j = 0; j < m; j++) rank += (cp[j] > v) || (cp[j] == v && ct[j] < t);
    p.tok_out[rank] = t; p.p_out[rank] = v;
  }
}

int launch_candidates(const float* logits, int n, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                      float repetition, float frequency, float presence, float temperature, int m,
                      float* probs_scratch, int32_t* tok_out, float* p_out)
{
  if (n < 1 || m < 1 || m > SMP_MAX_M) return set_error(CAI_ERR_INVALID, "candidates: %d tokens wanted from a row of %d (1..%d)", m, n, SMP_MAX_M);
  SampleParams p{logits, n, hist_ids, hist_counts, n_hist, repetition, frequency, presence, temperature, m, probs_scratch, tok_out, p_out};
  hipLaunchKernelGGL(candidates_kernel, dim3(1), dim3(SMP_T), 0, ctx().stream, p);
  return CAI_OK;
}

// host arrays in, host arrays out; the row itself is a device pointer
int run_candidates(const float* logits_dev, int n, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                   float repetition, float frequency, float presence, float temperature, int m,
                   int32_t* tokens_out, float* probs_out, int* count_out)
{
  Context& c = ctx();
  if (n_hist < 0 || (n_hist > 0 && (!hist_ids || !hist_counts))) return set_error(CAI_ERR_INVALID, "candidates: history of %d tokens without its arrays", n_hist);
  if (m > n) m = n;
  // stage_in: [history ids | history counts]; stage_out: [probabilities scratch n | tokens m | probabilities m]
  const size_t hist_b = (size_t)n_hist * sizeof(int32_t);
  int rc = ensure_stage(&c.stage_in, &c.stage_in_cap, 2 * hist_b + 16); if (rc) return rc;
  rc = ensure_stage(&c.stage_out, &c.stage_out_cap, ((size_t)n + 2 * (size_t)SMP_MAX_M) * 4); if (rc) return rc;
  int32_t* d_ids = (int32_t*)c.stage_in; int32_t* d_cnt = d_ids + n_hist;
  if (n_hist > 0) {
    CAI_HIP(hipMemcpyAsync(d_ids, hist_ids, hist_b, hipMemcpyHostToDevice, c.stream));
    CAI_HIP(hipMemcpyAsync(d_cnt, hist_counts, hist_b, hipMemcpyHostToDevice, c.stream));
  }
  float* scratch = (float*)c.stage_out;
  int32_t* d_tok = (int32_t*)(scratch + n); float* d_p = (float*)(d_tok + SMP_MAX_M);
  rc = launch_candidates(logits_dev, n, d_ids, d_cnt, n_hist, repetition, frequency, presence, temperature, m, scratch, d_tok, d_p);
  if (rc) return rc;
  CAI_HIP(hipMemcpyAsync(tokens_out, d_tok, (size_t)m * 4, hipMemcpyDeviceToHost, c.stream));
  CAI_HIP(hipMemcpyAsync(probs_out, d_p, (size_t)m * 4, hipMemcpyDeviceToHost, c.stream));
  CAI_HIP(hipStreamSynchronize(c.stream));
  if (count_out) *count_out = m;
  return CAI_OK;
}

}  // namespace cai

using namespace cai;

extern "C" int cai_sample_candidates(const float* logits, int n, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                                     float repetition, float frequency, float presence, float temperature, int m,
                                     int32_t* tokens_out, float* probs_out, int* count_out, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(logits && tokens_out && probs_out, "cai_sample_candidates: null argument");
  CAI_REQUIRE(n >= 1 && m >= 1 && m <= SMP_MAX_M, "cai_sample_candidates: %d candidates from a row of %d (1..%d)", m, n, SMP_MAX_M);
  Context& c = ctx();
  const float* row = logits;
  if (!(flags & CAI_X_DEVICE)) {
    // the row travels into a private device buffer behind the scratch areas run_candidates lays out
    int rc = ensure_stage(&c.stage_sample, &c.stage_sample_cap, (size_t)n * 4); if (rc) return rc;
    CAI_HIP(hipMemcpyAsync(c.stage_sample, logits, (size_t)n * 4, hipMemcpyHostToDevice, c.stream));
    row = (const float*)c.stage_sample;
  }
  return run_candidates(row, n, hist_ids, hist_counts, n_hist, repetition, frequency, presence, temperature, m, tokens_out, probs_out, count_out);
}
