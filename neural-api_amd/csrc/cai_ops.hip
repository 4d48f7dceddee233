// Elementwise layer math, block dequantization, embedding gather, arg-max and the MoE router for gfx950.
#include "cai_internal.hpp"
#include "cai_blocks_raw.hpp"
#include <string.h>
#include <math.h>

namespace cai {

__device__ __forceinline__ float wave_sum_all(float v)
{
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x112, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, true));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// ------------------------------------------------------------------------------------------
// Element (row, i) of a resident matrix, bit-exact to DecodeGGMLSpan (neural/neuralgguf.pas:1471-1523).
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ float f16_bits_to_float(uint16_t h) { return __half2float(__ushort_as_half(h)); }

__device__ float dequant_elem(int qtype, const uint8_t* data, const uint8_t* aux, const uint8_t* aux2, int64_t cols, int64_t row, int64_t i)
{
  switch (qtype) {
    case CAI_F32: return reinterpret_cast<const float*>(data)[row * cols + i];
    case CAI_F16: return f16_bits_to_float(reinterpret_cast<const uint16_t*>(data)[row * cols + i]);
    case CAI_I8ROW:  // code * Scales[row] (neural/neural.cl:1447-1470)
      return (float)reinterpret_cast<const int8_t*>(data)[row * cols + i] * reinterpret_cast<const float*>(aux)[row];
    case CAI_Q8_0: {  // x = d * q (neural/neuralgguf.pas:1487-1503)
      const float d = f16_bits_to_float(reinterpret_cast<const uint16_t*>(aux)[row * (cols >> 5) + (i >> 5)]);
      return d * (float)reinterpret_cast<const int8_t*>(data)[row * cols + i];
    }
    case CAI_Q4_0: {  // x = d * (nibble - 8); e<16 low nibble of byte e, else high nibble of byte e-16 (neuralgguf.pas:811-845)
      const int64_t blk = i >> 5; const int e = (int)(i & 31);
      const float d = f16_bits_to_float(reinterpret_cast<const uint16_t*>(aux)[row * (cols >> 5) + blk]);
      const uint8_t b = data[row * (cols >> 1) + blk * 16 + (e & 15)];
      const int nib = e < 16 ? (b & 15) : (b >> 4);
      return d * (float)(nib - 8);
    }
    case CAI_Q4_K: {  // x = (d*sc)*q - dmin*mn (neural/neuralgguf.pas:448-514)
      const uint8_t* blk = data + (row * (cols >> 8) + (i >> 8)) * 144;
      const int e = (int)(i & 255), c = e >> 6, hi = (e >> 5) & 1, idx = e & 31, j = 2 * c + hi;
      const float d = f16_bits_to_float(*reinterpret_cast<const uint16_t*>(blk));
      const float dmin = f16_bits_to_float(*reinterpret_cast<const uint16_t*>(blk + 2));
      const uint8_t* s = blk + 4;
      int sc, mn;
      if (j < 4) { sc = s[j] & 63; mn = s[j + 4] & 63; }
      else { sc = (s[j + 4] & 15) | ((s[j - 4] >> 2) & 0x30); mn = (s[j + 4] >> 4) | ((s[j] >> 2) & 0x30); }
      const uint8_t b = blk[16 + 32 * c + idx];
      const int q = hi ? (b >> 4) : (b & 15);
      const float dsc = d * (float)sc, dm = dmin * (float)mn;
      return dsc * (float)q - dm;
    }
    case CAI_Q6_K: {  // x = (d*scale[i/16]) * ((ql | qh<<4) - 32) (neural/neuralgguf.pas:639-717); resident as 192-byte ql|qh records, a scales plane and a d plane
      const int64_t b = row * (cols >> 8) + (i >> 8);
      const uint8_t* blk = data + b * 192;
      const int e = (int)(i & 255);
      const float d = f16_bits_to_float(reinterpret_cast<const uint16_t*>(aux2)[b]);
      const float dl = d * (float)reinterpret_cast<const int8_t*>(aux + b * 16)[e >> 4];
      const int lo = blk[(e >> 7) * 64 + (e & 63)];
      const int nib = (e & 127) < 64 ? (lo & 15) : (lo >> 4);
      const int hi2 = (blk[128 + (e >> 7) * 32 + (e & 31)] >> (2 * ((e & 127) >> 5))) & 3;
      return dl * (float)((nib | (hi2 << 4)) - 32);
    }
  }
  if (raw_block_type(qtype)) {   // resident as stored
    const int be = raw_block_elems(qtype);
    return raw_block_elem(qtype, data + (row * (cols / be) + i / be) * raw_block_bytes(qtype), (int)(i % be));
  }
  return 0.0f;
}

__global__ void dequant_rows_kernel(int qtype, const uint8_t* data, const uint8_t* aux, const uint8_t* aux2, int64_t cols, int64_t row0, int64_t n, float* out)
{
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  out[idx] = dequant_elem(qtype, data, aux, aux2, cols, row0 + idx / cols, idx % cols);
}

int launch_dequant_rows(const cai_qw_s* w, int64_t row0, int64_t n_rows, float* out)
{
  const int64_t n = n_rows * w->cols;
  hipLaunchKernelGGL(dequant_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx().stream,
                     w->qtype, w->data, w->aux, qw_aux2(w), w->cols, row0, n, out);
  return CAI_OK;
}

// Embedding gather (TNNetEmbedding; neural/neural.cl:1422-1470): Y[t] = W[token_t], dequantized.
__global__ void embed_kernel(int qtype, const uint8_t* data, const uint8_t* aux, const uint8_t* aux2, int64_t cols, const int32_t* tokens, float* out)
{
  const int t = blockIdx.y;
  const int64_t row = tokens[t];
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < cols; i += (int64_t)gridDim.x * blockDim.x)
    out[(int64_t)t * cols + i] = dequant_elem(qtype, data, aux, aux2, cols, row, i);
}

int launch_embed(const cai_qw_s* w, const int32_t* tokens_dev, int n_tokens, float* out)
{
  const int bx = (int)std::min<int64_t>((w->cols + 255) / 256, 64);
  hipLaunchKernelGGL(embed_kernel, dim3(bx, n_tokens), dim3(256), 0, ctx().stream, w->qtype, w->data, w->aux, qw_aux2(w), w->cols, tokens_dev, out);
  return CAI_OK;
}

// ---- GGUF block stream -> planes (Q8_0: 34-byte blocks, Q4_0: 18-byte blocks; neural/neuralgguf.pas:100-131) ----
__global__ void split_blocks_kernel(const uint8_t* raw, int block_bytes, int64_t n_blocks, uint8_t* qs, uint16_t* d)
{
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= n_blocks) return;
  const uint8_t* src = raw + b * block_bytes;
  d[b] = (uint16_t)(src[0] | (src[1] << 8));
  const int qb = block_bytes - 2;
  // 2-byte aligned source (block sizes are even): move halfwords
  const uint16_t* s16 = reinterpret_cast<const uint16_t*>(src + 2);
  uint16_t* d16 = reinterpret_cast<uint16_t*>(qs + b * qb);
  for (int i = 0; i < qb / 2; i++) d16[i] = s16[i];
}

// ---- Q6_K block stream (210 bytes: ql 128 | qh 64 | scales 16 | d 2, only 2-byte aligned) -> 192-byte ql|qh records, a plane
// of scales and a plane of d: every request of the kernels is then aligned (the raw stream costs a third of the rate) ----
__global__ void split_q6k_kernel(const uint8_t* raw, int64_t n_blocks, uint8_t* rec, uint8_t* sc, uint16_t* d)
{
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // one thread per halfword of a block
  const int64_t b = i / 105; const int h = (int)(i - b * 105);
  if (b >= n_blocks) return;
  const uint16_t v = reinterpret_cast<const uint16_t*>(raw)[i];
  if (h < 96) reinterpret_cast<uint16_t*>(rec)[b * 96 + h] = v;
  else if (h < 104) reinterpret_cast<uint16_t*>(sc)[b * 8 + (h - 96)] = v;
  else d[b] = v;
}
int launch_split_q6k(const uint8_t* raw, int64_t n_blocks, uint8_t* rec, uint8_t* sc, uint16_t* d)
{
  const int64_t n = n_blocks * 105;
  hipLaunchKernelGGL(split_q6k_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx().stream, raw, n_blocks, rec, sc, d);
  return CAI_OK;
}

int launch_split_blocks(const uint8_t* raw, int block_bytes, int64_t n_blocks, uint8_t* qs, uint16_t* d)
{
  hipLaunchKernelGGL(split_blocks_kernel, dim3((unsigned)((n_blocks + 255) / 256)), dim3(256), 0, ctx().stream, raw, block_bytes, n_blocks, qs, d);
  return CAI_OK;
}

// ---- TNNetTokenRMSNorm (neural/neural.cl:1047-1085): y = g * (x * rsqrt(mean(x^2) + eps)) ----
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* x, const float* gain, int n, float eps, float* y, int64_t x_stride, int64_t y_stride)
{
  const float* xr = x + (int64_t)blockIdx.x * x_stride;
  float* yr = y + (int64_t)blockIdx.x * y_stride;
  __shared__ float red[4];
  float ss = 0.0f;
  for_strided8(xr, threadIdx.x, n, 256, [&](float v, int) { ss = fmaf(v, v, ss); });
  ss = wave_sum_all(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float tot = (red[0] + red[1]) + (red[2] + red[3]);
  const float inv = 1.0f / sqrtf(tot / (float)n + eps);
  for_strided8(xr, gain, threadIdx.x, n, 256, [&](float v, float g, int i) { yr[i] = g * (v * inv); });
}

int launch_rmsnorm_strided(const float* x, const float* gain, int n, int n_tokens, float eps, float* y, int64_t x_stride, int64_t y_stride)
{
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(n_tokens), dim3(256), 0, ctx().stream, x, gain, n, eps, y, x_stride, y_stride);
  return CAI_OK;
}
// Two adjacent segments of every token row normalised in place by one launch (full-width q and k norms of OLMoE,
// neural/neuralpretrained.pas:16511-16530): work-group (t, 0) takes [0, n_a), (t, 1) takes [n_a, n_a + n_b).
__global__ __launch_bounds__(256) void rmsnorm_pair_kernel(float* x, const float* gain_a, int n_a, const float* gain_b, int n_b, float eps, int64_t stride)
{
  float* xr = x + (int64_t)blockIdx.x * stride + (blockIdx.y ? n_a : 0);
  const float* gain = blockIdx.y ? gain_b : gain_a;
  const int n = blockIdx.y ? n_b : n_a;
  __shared__ float red[4];
  float ss = 0.0f;
  for_strided8(xr, threadIdx.x, n, 256, [&](float v, int) { ss = fmaf(v, v, ss); });
  ss = wave_sum_all(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float tot = (red[0] + red[1]) + (red[2] + red[3]);
  const float inv = 1.0f / sqrtf(tot / (float)n + eps);
  for_strided8(xr, gain, threadIdx.x, n, 256, [&](float v, float g, int i) { xr[i] = g * (v * inv); });
}

int launch_rmsnorm_pair(float* x, const float* gain_a, int n_a, const float* gain_b, int n_b, int n_tokens, float eps, int64_t stride)
{
  hipLaunchKernelGGL(rmsnorm_pair_kernel, dim3(n_tokens, 2), dim3(256), 0, ctx().stream, x, gain_a, n_a, gain_b, n_b, eps, stride);
  return CAI_OK;
}
int launch_rmsnorm(const float* x, const float* gain, int n, int n_tokens, float eps, float* y)
{
  return launch_rmsnorm_strided(x, gain, n, n_tokens, eps, y, n, n);
}

// ---- TNNetRotaryEmbedding (neural/neural.cl:1517-1542), interleaved pairs, head-tiled theta ----
__global__ void rope_kernel(float* x, int n_heads, int head_dim, const int32_t* pos, const float* theta, int64_t token_stride)
{
  const int t = blockIdx.y;
  const int half = head_dim >> 1;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_heads * half) return;
  const int k = i % half;
  const float angle = (float)pos[t] * theta[k];
  float s, c; sincosf(angle, &s, &c);
  float* p = x + (int64_t)t * token_stride + (i / half) * head_dim + 2 * k;
  const float x0 = p[0], x1 = p[1];
  p[0] = c * x0 - s * x1;
  p[1] = s * x0 + c * x1;
}

int launch_rope(float* x, int n_heads, int head_dim, const int32_t* pos_dev, int, const float* theta, int n_tokens, int64_t token_stride)
{
  const int n = n_heads * (head_dim >> 1);
  hipLaunchKernelGGL(rope_kernel, dim3((n + 255) / 256, n_tokens), dim3(256), 0, ctx().stream, x, n_heads, head_dim, pos_dev, theta, token_stride);
  return CAI_OK;
}

// Host-side frequency table (neural/neural.cl:1510-1515): theta_k = base^(-2k/head_dim) in double, rounded once.
void rope_thetas(float base, int head_dim, std::vector<float>& out)
{
  out.resize(head_dim / 2);
  for (int k = 0; k < head_dim / 2; k++) out[k] = (float)pow((double)base, -2.0 * k / head_dim);
}

// The table under a long-context rule (neural/neuralpretrained.pas:633-668, rope_scaling): every rule here only changes the
// frequencies, so the kernels are the unscaled ones.  In double, rounded once.
//   linear (Position Interpolation): theta_k / factor
//   llama3: with r = original_ctx * theta_k / (2 pi) rotations over the training context: r > high_freq_factor keeps theta_k,
//           r < low_freq_factor takes theta_k / factor, between them the two are blended linearly in r (no output scale)
//   ntk:    base' = base * factor^(d / (d - 2)) (the static form of the dynamic rule at the full factor)
//   yarn:   pair k keeps theta_k below the correction dimension of high_freq_factor (= beta_fast) rotations, takes theta_k / factor
//           above that of low_freq_factor (= beta_slow), linear in k between (band edges floored / ceiled); the rotated q and k
//           are also multiplied by 0.1 ln(factor) + 1, which the session applies as its square on the attention scores
int rope_thetas_scaled(float base, int head_dim, int mode, float factor, int original_ctx, float low_freq_factor, float high_freq_factor, std::vector<float>& out)
{
  if (mode == CAI_ROPE_NONE) { rope_thetas(base, head_dim, out); return CAI_OK; }
  if (mode < CAI_ROPE_LINEAR || mode > CAI_ROPE_YARN) return set_error(CAI_ERR_UNSUPPORTED, "rope scaling: mode %d (0 none, 1 linear, 2 llama3, 3 ntk, 4 yarn)", mode);
  if (!(factor >= 1.0f)) return set_error(CAI_ERR_INVALID, "rope scaling: factor must be >= 1, got %g", (double)factor);
  if ((mode == CAI_ROPE_LLAMA3 || mode == CAI_ROPE_YARN) && (original_ctx <= 0 || !(high_freq_factor > low_freq_factor) || !(low_freq_factor > 0.0f)))
    return set_error(CAI_ERR_INVALID, "rope scaling: llama3 / yarn need original_ctx > 0 and high_freq_factor > low_freq_factor > 0 (got %d, %g, %g)", original_ctx, (double)high_freq_factor, (double)low_freq_factor);
  if (mode == CAI_ROPE_NTK && head_dim <= 2) return set_error(CAI_ERR_INVALID, "rope scaling: ntk needs a head wider than 2");
  out.resize(head_dim / 2);
  const double two_pi = 6.283185307179586476925286766559;
  double ylow = 0.0, yhigh = 1.0;
  if (mode == CAI_ROPE_YARN) {
    const double lb = 2.0 * log((double)base);
    ylow = std::max(0.0, floor(head_dim * log((double)original_ctx / ((double)high_freq_factor * two_pi)) / lb));
    yhigh = std::min((double)(head_dim - 1), ceil(head_dim * log((double)original_ctx / ((double)low_freq_factor * two_pi)) / lb));
    if (yhigh == ylow) yhigh += 0.001;
  }
  for (int k = 0; k < head_dim / 2; k++) {
    const double th = pow((double)base, -2.0 * k / head_dim);
    double v = th / (double)factor;
    if (mode == CAI_ROPE_NTK) v = pow((double)base * pow((double)factor, (double)head_dim / (head_dim - 2.0)), -2.0 * k / head_dim);
    if (mode == CAI_ROPE_YARN) {
      const double ramp = std::min(1.0, std::max(0.0, ((double)k - ylow) / (yhigh - ylow)));
      v = (th / (double)factor) * ramp + th * (1.0 - ramp);
    }
    if (mode == CAI_ROPE_LLAMA3) {
      const double r = (double)original_ctx * th / two_pi;
      if (r > (double)high_freq_factor) v = th;
      else if (r >= (double)low_freq_factor) {
        const double smooth = (r - (double)low_freq_factor) / ((double)high_freq_factor - (double)low_freq_factor);
        v = (1.0 - smooth) * th / (double)factor + smooth * th;
      }
    }
    out[k] = (float)v;
  }
  return CAI_OK;
}

__global__ void add_kernel(float* x, const float* y, int64_t n)
{
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] += y[i];
}
int launch_add(float* x, const float* y, int64_t n)
{
  hipLaunchKernelGGL(add_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx().stream, x, y, n);
  return CAI_OK;
}

// x[t][i] += sum_j gate[t][j] * part[t][j][i]   (gate-weighted expert mixture, neural/neural.cl:2738-2751)
__global__ void moe_combine_kernel(float* x, const float* part, const float* gate, int k, int n)
{
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float acc = 0.0f;
  const float xv = x[(int64_t)t * n + i];
  for (int j0 = 0; j0 < k; j0 += 8) {      // eight experts' values are requested together; the sum keeps the expert order
    float pv[8], gv[8];
#pragma unroll
    for (int u = 0; u < 8; u++) { const int j = min(j0 + u, k - 1); pv[u] = part[((int64_t)t * k + j) * n + i]; gv[u] = gate[t * k + j]; }
#pragma unroll
    for (int u = 0; u < 8; u++) if (j0 + u < k) acc = fmaf(gv[u], pv[u], acc);
  }
  x[(int64_t)t * n + i] = xv + acc;
}
int launch_moe_combine(float* x, const float* part, const float* gate, int k, int n, int n_tokens)
{
  hipLaunchKernelGGL(moe_combine_kernel, dim3((n + 255) / 256, n_tokens), dim3(256), 0, ctx().stream, x, part, gate, k, n);
  return CAI_OK;
}

// Gathered down projection and the gate-weighted mixture of a token in ONE launch (Q8_0 expert bank, up to 8 selected experts):
// a wave takes R output rows for ALL selected experts - the R x k weight rows (a lane 16 values of each per 1024 columns), the
// k SwiGLU rows and the gates are requested together, one round trip behind the expert ids - and adds
// sum_j gate_j * (row of expert j . mid_j) to the residual row in place (neural/neuralpretrained.pas:15372-15388).  Takes the
// place of the gathered matrix-vector launch, its k partial rows and the mixture launch.
template <int R>
__global__ __launch_bounds__(256) void moe_down_mix_kernel(const int8_t* wq, const __half* wsc, const int bank_experts, const int dm, const int cols,
                                                           const float* mid, const int32_t* experts, const float* gates, const int k, float* x)
{
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int row0 = (blockIdx.x * 4 + w) * R;
  if (row0 >= dm) return;               // (no barrier in this kernel)
  int e[8]; float g[8];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const int jj = min(j, k - 1);
    e[j] = min(max(experts[jj], 0), bank_experts - 1);      // an id outside the bank (a router fed NaN) must not address memory
    g[j] = j < k ? gates[jj] : 0.0f;
  }
  const int nblk = cols >> 5;
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = 0.0f;
  for (int c0 = 0; c0 < cols; c0 += 1024) {
    const bool on = c0 + 16 * lane < cols;
    const int col = on ? c0 + 16 * lane : 0;
    uint4 q[8][R]; float sc[8][R]; float4 xv[8][4];
#pragma unroll
    for (int j = 0; j < 8; j++) {
#pragma unroll
      for (int r = 0; r < R; r++) {
        const int64_t row = (int64_t)e[j] * dm + min(row0 + r, dm - 1);
        q[j][r] = *reinterpret_cast<const uint4*>(wq + row * cols + col);
        sc[j][r] = __half2float(wsc[row * nblk + (col >> 5)]);
      }
#pragma unroll
      for (int u = 0; u < 4; u++) xv[j][u] = reinterpret_cast<const float4*>(mid + (int64_t)min(j, k - 1) * cols + col)[u];
    }
    if (on) {
#pragma unroll
      for (int j = 0; j < 8; j++)
#pragma unroll
        for (int r = 0; r < R; r++) {
          const int c4[4] = {(int)q[j][r].x, (int)q[j][r].y, (int)q[j][r].z, (int)q[j][r].w};
          float d = 0.0f;
#pragma unroll
          for (int u = 0; u < 4; u++) {
            d = fmaf(xv[j][u].x, (float)((c4[u] << 24) >> 24), d); d = fmaf(xv[j][u].y, (float)((c4[u] << 16) >> 24), d);
            d = fmaf(xv[j][u].z, (float)((c4[u] << 8) >> 24), d); d = fmaf(xv[j][u].w, (float)(c4[u] >> 24), d);
          }
          acc[r] = fmaf(g[j] * sc[j][r], d, acc[r]);
        }
    }
  }
#pragma unroll
  for (int r = 0; r < R; r++) {
    float a = acc[r];
    for (int m = 32; m >= 1; m >>= 1) a += __shfl_xor(a, m, 64);
    if (lane == 0 && row0 + r < dm) x[row0 + r] += a;
  }
}
bool moe_down_mix_supported(const cai_qw_s* w, int dm, int k)
{
  static const bool off = []() { const char* e = getenv("CAIHIP_MOE_DOWN_LAUNCHES"); return e && e[0] == '1'; }();   // keep the two launches
  return !off && w->qtype == CAI_Q8_0 && !w->bias && k >= 1 && k <= 8 && dm > 0 && w->rows % dm == 0 && w->cols % 32 == 0;
}
int launch_moe_down_mix(const cai_qw_s* w, int dm, const float* mid, const int32_t* experts, const float* gates, int k, float* x)
{
  if (!moe_down_mix_supported(w, dm, k)) return set_error(CAI_ERR_UNSUPPORTED, "moe: the one-launch down projection takes a Q8_0 bank and up to 8 selected experts");
  if ((reinterpret_cast<uintptr_t>(mid) | reinterpret_cast<uintptr_t>(w->data)) & 15) return set_error(CAI_ERR_INVALID, "moe: rows must be 16-byte aligned");
  constexpr int R = 2;
  hipLaunchKernelGGL(moe_down_mix_kernel<R>, dim3((unsigned)((dm + 4 * R - 1) / (4 * R))), dim3(256), 0, ctx().stream, (const int8_t*)w->data, (const __half*)w->aux,
                     (int)(w->rows / dm), dm, (int)w->cols, mid, experts, gates, k, x);
  return CAI_OK;
}

// ---- ArgMaxRow (neural/neuralchatengine.pas:683-697): strict >, lowest index wins ties ----
// Two stages: work-groups scan 4096-element slices, then one work-group folds the slice winners.
__device__ __forceinline__ bool argmax_better(float v, int i, float bv, int bi) { return bi < 0 || v > bv || (v == bv && i < bi); }

__global__ __launch_bounds__(256) void argmax_stage1(const float* x, int n, float* pv, int32_t* pi, int n_slices)
{
  const int row = blockIdx.y, slice = blockIdx.x;
  const float* xr = x + (int64_t)row * n;
  float best = 0.0f; int bi = -1;
  const int i0 = slice * 4096, i1 = min(n, i0 + 4096);
  if (i0 < i1) for_strided8(xr + i0, threadIdx.x, i1 - i0, 256, [&](float v, int i) { if (bi < 0 || v > best) { best = v; bi = i0 + i; } });
  __shared__ float sv[256]; __shared__ int si[256];
  sv[threadIdx.x] = best; si[threadIdx.x] = bi;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) {
      const float ov = sv[threadIdx.x + s]; const int oi = si[threadIdx.x + s];
      if (oi >= 0 && argmax_better(ov, oi, sv[threadIdx.x], si[threadIdx.x])) { sv[threadIdx.x] = ov; si[threadIdx.x] = oi; }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) { pv[row * n_slices + slice] = sv[0]; pi[row * n_slices + slice] = si[0]; }
}

__global__ __launch_bounds__(64) void argmax_stage2(const float* pv, const int32_t* pi, int n_slices, int32_t* out)
{
  const int row = blockIdx.x;
  float best = 0.0f; int bi = -1;
  for (int s = threadIdx.x; s < n_slices; s += 64) {
    const float v = pv[row * n_slices + s]; const int i = pi[row * n_slices + s];
    if (i >= 0 && argmax_better(v, i, best, bi)) { best = v; bi = i; }
  }
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off); const int oi = __shfl_xor(bi, off);
    if (oi >= 0 && argmax_better(ov, oi, best, bi)) { best = ov; bi = oi; }
  }
  if (threadIdx.x == 0) out[row] = bi < 0 ? 0 : bi;
}

int launch_argmax(const float* x, int n, int n_rows, int32_t* out, float* scratch_v, int32_t* scratch_i)
{
  const int n_slices = (n + 4095) / 4096;
  hipLaunchKernelGGL(argmax_stage1, dim3(n_slices, n_rows), dim3(256), 0, ctx().stream, x, n, scratch_v, scratch_i, n_slices);
  hipLaunchKernelGGL(argmax_stage2, dim3(n_rows), dim3(64), 0, ctx().stream, scratch_v, scratch_i, n_slices, out);
  return CAI_OK;
}
int argmax_scratch_entries(int n, int n_rows) { return (n + 4095) / 4096 * n_rows; }

// ---- arg-max for callers that cannot allocate (cai_argmax_noalloc) ----
// The slice winners of stage 1 (one float + one index per 4096 elements) go to a file-scope device array instead of the
// staging buffer cai_argmax grows on demand.  Every GPU holds its own copy of the array at its own address: the address is
// looked up once per device, with that device current, and host code only ever uses that pointer.
constexpr int NOALLOC_MAX_SLICES = 1024;                     // rows of up to 4096 * 1024 = 4 194 304 elements
constexpr int NOALLOC_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char scratch[NOALLOC_MAX_SLICES * 8];
static void* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {nullptr};

int noalloc_setup(int device)
{
  if (device < 0 || device >= NOALLOC_MAX_DEVICES) return set_error(CAI_ERR_INVALID, "device ordinal %d outside 0..%d", device, NOALLOC_MAX_DEVICES - 1);
  if (g_scratch_ptr[device]) return CAI_OK;
  void* ptr = nullptr;
  CAI_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  g_scratch_ptr[device] = ptr;
  return CAI_OK;
}

// ---- router: TNNetPointwiseSoftMax (neural/neural.cl:1594-1647) + TNNetTopKGate ----
// One wave per token; lane i owns experts i, i+64, ...  Selection is k rounds of a wave-wide arg-max in which the
// larger probability wins and, between equals, the lower expert index (the reference scans upwards with '>').
constexpr int ROUTER_MAX_PER_LANE = 8;   // up to 512 experts
// Selection key of a probability: larger key = selected earlier.  A total order whatever the value: lanes that hold no expert
// get 0, a NaN (a poisoned activation row reaches the router as NaN logits) ranks below every number, and probabilities are
// non-negative, so their bit patterns order like their values.  With a total order the k selected experts are always k
// distinct ids inside [0, n); the gates still carry the NaN to the outputs.
__device__ __forceinline__ uint32_t router_key(float p, bool candidate)
{
  if (!candidate) return 0u;
  if (!(p == p)) return 1u;
  return __builtin_bit_cast(uint32_t, fmaxf(p, 0.0f)) + 2u;
}
// Soft-max over n <= 64 logits and the k largest probabilities, by ONE wave (lane i owns expert i and brings its logit): every lane ranks its own
// probability against the 64 broadcast ones (larger first, lower index between equals) - a permutation of 0..63 - and the lanes
// of rank 0..k-1 are the selection, in order.  Returns the probability of the lane's expert; lane j < k gets the j-th selected
// expert and its gate (divided by the sum of the k selected when renorm is set).
__device__ __forceinline__ float router_select64(float logit, int n, int k, int renorm, int lane, int& expert_j, float& gate_j)
{
  float v = lane < n ? logit : -3.0e38f;
  float mx = v;
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  float a = v - mx; a = a > 4000.0f ? 4000.0f : (a < -4000.0f ? -4000.0f : a);
  v = lane < n ? expf(a) : 0.0f;
  float tot = v;
  for (int m = 32; m >= 1; m >>= 1) tot += __shfl_xor(tot, m, 64);
  const float inv = tot > 0.0f ? 1.0f / tot : 1.0f;
  v *= inv;
  const float pv = lane < n ? v : -1.0f;      // -1 marks "not a candidate"
  const uint32_t key = router_key(pv, lane < n);
  int rank = 0;
  for (int j = 0; j < 64; j++) {
    const uint32_t o = (uint32_t)__builtin_amdgcn_readlane((int)key, j);
    rank += (o > key || (o == key && j < lane)) ? 1 : 0;
  }
  float sum = 0.0f, mine = 0.0f;
  expert_j = 0;
  for (int j = 0; j < k; j++) {
    const int src = __ffsll((unsigned long long)__ballot(rank == j)) - 1;
    const float bv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, pv), src));
    if (lane == j) { mine = bv; expert_j = src; }
    sum += bv;
  }
  gate_j = renorm ? (sum > 0.0f ? mine * (1.0f / sum) : 0.0f) : mine;
  return v;
}
__global__ __launch_bounds__(64) void router_topk_kernel(const float* logits, int n, int k, int renorm, int n_tokens, int32_t* expert_out, float* gate_out, float* probs)
{
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* x = logits + (int64_t)t * n;
  if (n <= 64) {     // one expert per lane
    int ej; float gj;
    const float pr = router_select64(lane < n ? x[lane] : 0.0f, n, k, renorm, lane, ej, gj);
    if (lane < n) probs[(int64_t)t * n + lane] = pr;
    if (lane < k) { expert_out[t * k + lane] = ej; gate_out[t * k + lane] = gj; }
    return;
  }
  float v[ROUTER_MAX_PER_LANE];
  float mx = -3.0e38f;
#pragma unroll
  for (int i = 0; i < ROUTER_MAX_PER_LANE; i++) {
    const int c = lane + 64 * i;
    v[i] = c < n ? x[c] : -3.0e38f;
    mx = fmaxf(mx, v[i]);
  }
  for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
  float tot = 0.0f;
#pragma unroll
  for (int i = 0; i < ROUTER_MAX_PER_LANE; i++) {
    const int c = lane + 64 * i;
    float a = v[i] - mx; a = a > 4000.0f ? 4000.0f : (a < -4000.0f ? -4000.0f : a);
    v[i] = c < n ? expf(a) : 0.0f;
    tot += v[i];
  }
  for (int m = 32; m >= 1; m >>= 1) tot += __shfl_xor(tot, m, 64);
  const float inv = tot > 0.0f ? 1.0f / tot : 1.0f;
#pragma unroll
  for (int i = 0; i < ROUTER_MAX_PER_LANE; i++) {
    const int c = lane + 64 * i;
    v[i] *= inv;
    if (c < n) probs[(int64_t)t * n + c] = v[i]; else v[i] = -1.0f;   // -1 marks "not a candidate"
  }
  float sum = 0.0f, mine = 0.0f;   // lane j keeps the j-th selected gate
  uint32_t key[ROUTER_MAX_PER_LANE];
#pragma unroll
  for (int i = 0; i < ROUTER_MAX_PER_LANE; i++) key[i] = router_key(v[i], lane + 64 * i < n);
  for (int j = 0; j < k; j++) {   // k <= n: an expert that has not been taken (key >= 1) exists in every round
    uint32_t bk = 0u; float bv = 0.0f; int bc = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < ROUTER_MAX_PER_LANE; i++)
      if (key[i] > bk) { bk = key[i]; bv = v[i]; bc = lane + 64 * i; }   // ascending index inside the lane: '>' keeps the first
    for (int m = 32; m >= 1; m >>= 1) {
      const uint32_t ok = __shfl_xor(bk, m, 64); const float ov = __shfl_xor(bv, m, 64); const int oc = __shfl_xor(bc, m, 64);
      if (ok > bk || (ok == bk && oc < bc)) { bk = ok; bv = ov; bc = oc; }
    }
    if ((bc & 63) == lane) {
#pragma unroll
      for (int i = 0; i < ROUTER_MAX_PER_LANE; i++) if (bc == lane + 64 * i) key[i] = 0u;   // taken
    }
    if (lane == (j & 63)) { mine = bv; expert_out[t * k + j] = bc; }
    sum += bv;
  }
  if (lane < k) gate_out[t * k + lane] = renorm ? (sum > 0.0f ? mine * (1.0f / sum) : 0.0f) : mine;
}

int launch_router_topk(const float* logits, int n, int k, int renorm, int n_tokens, int32_t* expert_out, float* gate_out, float* probs_scratch)
{
  if (n < 1 || n > 64 * ROUTER_MAX_PER_LANE || k < 1 || k > 64 || k > n) return set_error(CAI_ERR_UNSUPPORTED, "router: %d experts, top-%d (supported: up to %d experts, k <= 64)", n, k, 64 * ROUTER_MAX_PER_LANE);
  hipLaunchKernelGGL(router_topk_kernel, dim3(n_tokens), dim3(64), 0, ctx().stream, logits, n, k, renorm, n_tokens, expert_out, gate_out, probs_scratch);
  return CAI_OK;
}

// The router of up to 64 experts in ONE launch: a work-group of four waves per four experts and token (one work-group for all
// the rows measured slower than the two launches it replaced: a single CU streams the 128 KB of a 64 x 2048 router at about
// 20 GB/s).  Every wave sums the squares of the row itself (no meeting before the products), takes one Q8_0 router row (a lane
// one 32-value block per 2048 columns; the factor 1 / rms multiplies the finished sum) and stores its logit at agent scope; the
// work-group that arrives last (wrapping counter per token, the hand-over of the attention merge: agent-scope stores
// acknowledged under vmcnt(0), work-group barrier, agent-scope increment, agent-scope loads) selects (router_select64).  Takes the
// place of the matrix-vector launch and the selection launch of a decode step (TNNetPointwiseSoftMax + TNNetTopKGate behind the
// router's TNNetPointwiseConvLinear, neural/neuralpretrained.pas:15331-15348).
#if defined(__HIP_DEVICE_COMPILE__) && !defined(CAI_MERGE_RELACQ) && !defined(__gfx950__) && !defined(__gfx942__)
#error "router_fused_kernel: the relaxed hand-over is only valid on gfx942 / gfx950; build with -DCAI_MERGE_RELACQ"
#endif
__global__ __launch_bounds__(256) void router_fused_kernel(const float* x, const long long x_stride, const float* gain, const float eps,
                                                           const int8_t* wq, const __half* wsc, const int n, const int cols, const int k, const int renorm,
                                                           float* logits_out, int32_t* expert_out, float* gate_out, float* probs, unsigned* counters)
{
  __shared__ int s_is_last;
  const int t = blockIdx.y, tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int r_own = blockIdx.x * 4 + w, r = min(r_own, n - 1);
  const float* xb = x + (int64_t)t * x_stride;
  const int nblk = cols >> 5;
  float acc = 0.0f, ss = 0.0f;
  for (int c0 = 0; c0 < nblk; c0 += 64) {
    const bool on = c0 + lane < nblk;
    const int blk = on ? c0 + lane : nblk - 1;
    const uint4* src = reinterpret_cast<const uint4*>(wq + (int64_t)r * cols + 32 * blk);
    const uint4 q0 = src[0], q1 = src[1];
    const float sc = __half2float(wsc[(int64_t)r * nblk + blk]);
    const uint32_t wd[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    float d = 0.0f;
#pragma unroll
    for (int q = 0; q < 8; q++) {
      const float4 v = reinterpret_cast<const float4*>(xb + 32 * blk)[q], g = reinterpret_cast<const float4*>(gain + 32 * blk)[q];
      const float xv[4] = {on ? v.x : 0.0f, on ? v.y : 0.0f, on ? v.z : 0.0f, on ? v.w : 0.0f};
      const int c4 = (int)wd[q];
      ss = fmaf(xv[0], xv[0], ss); ss = fmaf(xv[1], xv[1], ss); ss = fmaf(xv[2], xv[2], ss); ss = fmaf(xv[3], xv[3], ss);
      d = fmaf(g.x * xv[0], (float)((c4 << 24) >> 24), d); d = fmaf(g.y * xv[1], (float)((c4 << 16) >> 24), d);
      d = fmaf(g.z * xv[2], (float)((c4 << 8) >> 24), d); d = fmaf(g.w * xv[3], (float)(c4 >> 24), d);
    }
    acc = fmaf(d, sc, acc);
  }
  for (int m = 32; m >= 1; m >>= 1) { ss += __shfl_xor(ss, m, 64); acc += __shfl_xor(acc, m, 64); }
  const float logit = acc * (1.0f / sqrtf(ss / (float)cols + eps));
  if (lane == 0 && r_own < n) __hip_atomic_store(logits_out + (int64_t)t * n + r_own, logit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): the logit store has been acknowledged
  __syncthreads();
  if (tid == 0)
#ifdef CAI_MERGE_RELACQ
    s_is_last = __builtin_amdgcn_atomic_inc32(counters + t, gridDim.x - 1, __ATOMIC_RELEASE, "agent") == gridDim.x - 1;
#else
    s_is_last = __builtin_amdgcn_atomic_inc32(counters + t, gridDim.x - 1, __ATOMIC_RELAXED, "agent") == gridDim.x - 1;
#endif
  __syncthreads();
  if (!s_is_last || w != 0) return;
#ifdef CAI_MERGE_RELACQ
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#endif
  const float lg = __hip_atomic_load(logits_out + (int64_t)t * n + min(lane, n - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  int ej; float gj;
  const float pr = router_select64(lg, n, k, renorm, lane, ej, gj);
  if (lane < n) probs[(int64_t)t * n + lane] = pr;
  if (lane < k) { expert_out[t * k + lane] = ej; gate_out[t * k + lane] = gj; }
}

bool router_fused_supported(const cai_qw_s* w, int k)
{
  static const bool off = []() { const char* e = getenv("CAIHIP_ROUTER_LAUNCHES"); return e && e[0] == '1'; }();   // keep the two launches
  return !off && w->qtype == CAI_Q8_0 && !w->bias && w->rows >= 1 && w->rows <= 64 && k >= 1 && k <= w->rows && w->cols % 32 == 0;
}
int launch_router_fused(const cai_qw_s* w, const float* x, int64_t x_stride, const float* gain, float eps, int k, int renorm, int n_tokens,
                        float* logits_out, int32_t* expert_out, float* gate_out, float* probs_scratch, unsigned* counters)
{
  if (!router_fused_supported(w, k) || !gain || !counters) return set_error(CAI_ERR_UNSUPPORTED, "router: the one-launch form takes a Q8_0 router of up to 64 experts with a norm gain");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gain) | (uintptr_t)(x_stride * 4)) & 15) return set_error(CAI_ERR_INVALID, "router: activation rows and gain must be 16-byte aligned");
  hipLaunchKernelGGL(router_fused_kernel, dim3((unsigned)((w->rows + 3) / 4), n_tokens), dim3(256), 0, ctx().stream, x, (long long)x_stride, gain, eps, (const int8_t*)w->data, (const __half*)w->aux,
                     (int)w->rows, (int)w->cols, k, renorm, logits_out, expert_out, gate_out, probs_scratch, counters);
  return CAI_OK;
}

}  // namespace cai

// ------------------------------------------------------------------------------------------
// C ABI: standalone layer ops
// ------------------------------------------------------------------------------------------
using namespace cai;

namespace {
// Stages a host input on the device when needed; returns the device pointer to use.
int stage_input(const void* p, size_t bytes, int is_dev, const void** dev)
{
  Context& c = ctx();
  if (is_dev) { *dev = p; return CAI_OK; }
  const int rc = ensure_stage(&c.stage_in, &c.stage_in_cap, bytes); if (rc) return rc;
  CAI_HIP(hipMemcpyAsync(c.stage_in, p, bytes, hipMemcpyHostToDevice, c.stream));
  *dev = c.stage_in;
  return CAI_OK;
}
int stage_output(void* p, size_t bytes, int is_dev, void** dev)
{
  Context& c = ctx();
  if (is_dev) { *dev = p; return CAI_OK; }
  const int rc = ensure_stage(&c.stage_out, &c.stage_out_cap, bytes); if (rc) return rc;
  *dev = c.stage_out;
  return CAI_OK;
}
int finish_output(void* host, const void* dev, size_t bytes, int is_dev)
{
  Context& c = ctx();
  if (!is_dev) CAI_HIP(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, c.stream));
  CAI_HIP(hipStreamSynchronize(c.stream));
  return CAI_OK;
}
}  // namespace

extern "C" int cai_rmsnorm(const float* x, const float* gain_host, int n, int n_tokens, float eps, float* y, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(x && gain_host && y && n > 0 && n_tokens > 0, "cai_rmsnorm: bad argument");
  Context& c = ctx();
  const size_t bytes = (size_t)n * n_tokens * 4;
  float* d_gain = nullptr;
  CAI_HIP(hipMalloc(&d_gain, (size_t)n * 4));
  CAI_HIP(hipMemcpyAsync(d_gain, gain_host, (size_t)n * 4, hipMemcpyHostToDevice, c.stream));
  const void* dx; void* dy; int rc;
  if ((rc = stage_input(x, bytes, flags & CAI_X_DEVICE, &dx))) { (void)hipFree(d_gain); return rc; }
  if ((rc = stage_output(y, bytes, flags & CAI_Y_DEVICE, &dy))) { (void)hipFree(d_gain); return rc; }
  launch_rmsnorm((const float*)dx, d_gain, n, n_tokens, eps, (float*)dy);
  rc = finish_output(y, dy, bytes, flags & CAI_Y_DEVICE);
  (void)hipFree(d_gain);
  return rc;
}

extern "C" int cai_rope(float* x, int n_heads, int head_dim, int pos, float theta_base, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(x && n_heads > 0 && head_dim >= 2 && !(head_dim & 1) && head_dim <= 512, "cai_rope: bad argument");
  Context& c = ctx();
  std::vector<float> th; rope_thetas(theta_base, head_dim, th);
  float* d_th = reinterpret_cast<float*>(c.d_small + 16);
  static_assert(sizeof(float) == sizeof(int32_t), "");
  c.h_small[0] = pos;
  memcpy(c.h_small + 16, th.data(), th.size() * 4);   // h_small/d_small hold 16 ints + 256 floats
  CAI_HIP(hipMemcpyAsync(c.d_small, c.h_small, (16 + th.size()) * 4, hipMemcpyHostToDevice, c.stream));
  const size_t bytes = (size_t)n_heads * head_dim * 4;
  const int dev = (flags & (CAI_X_DEVICE | CAI_Y_DEVICE)) != 0;
  float* dx = x;
  if (!dev) {
    const int rc = ensure_stage(&c.stage_in, &c.stage_in_cap, bytes); if (rc) return rc;
    CAI_HIP(hipMemcpyAsync(c.stage_in, x, bytes, hipMemcpyHostToDevice, c.stream));
    dx = (float*)c.stage_in;
  }
  launch_rope(dx, n_heads, head_dim, c.d_small, 0, d_th, 1, 0);
  return finish_output(x, dx, bytes, dev);
}

extern "C" int cai_swiglu(const float* x, int half, int n_tokens, float* y, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(x && y && half > 0 && n_tokens > 0, "cai_swiglu: bad argument");
  const size_t ob = (size_t)half * n_tokens * 4;
  const void* dx; void* dy; int rc;
  if ((rc = stage_input(x, 2 * ob, flags & CAI_X_DEVICE, &dx))) return rc;
  if ((rc = stage_output(y, ob, flags & CAI_Y_DEVICE, &dy))) return rc;
  launch_swiglu((const float*)dx, half, n_tokens, (float*)dy);
  return finish_output(y, dy, ob, flags & CAI_Y_DEVICE);
}

extern "C" int cai_argmax(const float* x, int n, int32_t* index_out, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(x && index_out && n > 0, "cai_argmax: bad argument");
  Context& c = ctx();
  const void* dx; int rc;
  if ((rc = stage_input(x, (size_t)n * 4, flags & CAI_X_DEVICE, &dx))) return rc;
  const int ne = argmax_scratch_entries(n, 1);
  void* scr; if ((rc = stage_output(nullptr, (size_t)ne * 8, 0, &scr))) return rc;
  launch_argmax((const float*)dx, n, 1, c.d_small, (float*)scr, (int32_t*)scr + ne);
  CAI_HIP(hipMemcpyAsync(c.h_small, c.d_small, 4, hipMemcpyDeviceToHost, c.stream));
  CAI_HIP(hipStreamSynchronize(c.stream));
  *index_out = c.h_small[0];
  return CAI_OK;
}

// No hipMalloc, no hipFree, no copy, no wait: two launches on the library stream.  Stage 1 writes every slot stage 2 reads
// (slices 0 .. ceil(n / 4096) - 1), so nothing in the array has to be cleared between calls; calls that overlap on one GPU
// would share the array and race.
extern "C" int cai_argmax_noalloc(const float* x_dev, int n, int32_t* index_out_dev)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(x_dev && index_out_dev && n > 0, "cai_argmax_noalloc: bad argument");
  if (n > 4096 * NOALLOC_MAX_SLICES)
    return set_error(CAI_ERR_INVALID, "cai_argmax_noalloc: %d elements exceed the fixed scratch of %d (use cai_argmax)", n, 4096 * NOALLOC_MAX_SLICES);
  void* ptr = g_scratch_ptr[ctx().device];
  if (!ptr) return set_error(CAI_ERR_STATE, "cai_argmax_noalloc: scratch address of device %d was not resolved at cai_init", ctx().device);
  const int ne = argmax_scratch_entries(n, 1);
  launch_argmax(x_dev, n, 1, index_out_dev, (float*)ptr, (int32_t*)ptr + ne);
  CAI_HIP(hipGetLastError());
  return CAI_OK;
}

extern "C" int cai_router_topk(const float* logits, int n, int k, int renorm, int32_t* expert_out, float* gate_out, int flags)
{
  CAI_ENTER();
  CAI_READY();
  CAI_REQUIRE(logits && expert_out && gate_out && n > 0 && k > 0 && k <= n && k <= 64, "cai_router_topk: bad argument");
  Context& c = ctx();
  const void* dx; void* dscr; int rc;
  if ((rc = stage_input(logits, (size_t)n * 4, flags & CAI_X_DEVICE, &dx))) return rc;
  if ((rc = stage_output(nullptr, (size_t)n * 4, 0, &dscr))) return rc;
  int32_t* d_e = c.d_small; float* d_g = reinterpret_cast<float*>(c.d_small + 64);
  if ((rc = launch_router_topk((const float*)dx, n, k, renorm, 1, d_e, d_g, (float*)dscr))) return rc;
  CAI_HIP(hipMemcpyAsync(c.h_small, c.d_small, 128 * 4, hipMemcpyDeviceToHost, c.stream));
  CAI_HIP(hipStreamSynchronize(c.stream));
  for (int j = 0; j < k; j++) { expert_out[j] = c.h_small[j]; memcpy(&gate_out[j], &c.h_small[64 + j], 4); }
  return CAI_OK;
}
