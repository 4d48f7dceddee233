// Multi-token (prefill) linear layer on the matrix cores of gfx950.
//
// A prompt is a genuine dense contraction: Y[t][r] = sum_k W[r][k] X[t][k] for T tokens at once, so every weight
// block is read once per 128 tokens instead of once per token.  The reference has no such path (its prefill is
// token-at-a-time, neural/neuralchatengine.pas:1466-1470); the requirement is that the result equals T
// single-token linear layers, so the kernel keeps fp32-level accuracy instead of rounding operands to half:
//   * the block INTEGERS q (nibbles 0..15) are exact in f16 and go to the MFMA as they are;
//   * each activation is scaled per token by a power of two and split x = hi + lo into two f16 (22 bits);
//   * P = sum_{k in block} q_k x_k comes out of v_mfma_f32_32x32x8_f16 with fp32 accumulation;
//   * the block scales are applied in fp32 afterwards: Y += (d*sc) * P - (dmin*mn) * sum_{k in block} x_k
//     (Q4_K, neural/neuralgguf.pas:472-514).
#include "cai_internal.hpp"
#include "cai_gemv_common.hpp"
#include <algorithm>

namespace cai {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int PF_TOK = 128;   // tokens per work-group tile
constexpr int PF_KC = 64;     // reduction chunk: one 32-byte Q4_K quant chunk = two sub-blocks
constexpr int PF_LDK = PF_KC + 4;   // padded LDS row (halfs)

// ------------------------------------------------------------------------------------------
// Activation pre-pass (one work-group per token): optional RMSNorm (neural/neural.cl:1047-1085), then
//   s = 2^e with max|x|*s in [2^13, 2^14),  hi = f16(x*s),  lo = f16(x*s - hi),  sx[b] = sum of x over 32-block b.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void xprep_kernel(const float* x, int64_t x_stride, const float* gain, float eps, int K,
                                                    _Float16* hi, _Float16* lo, float* sx, float* sinv)
{
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float* xr = x + (int64_t)t * x_stride;
  __shared__ float red[4];
  __shared__ float s_scale;
  float inv = 1.0f;
  if (gain) {
    float ss = 0.0f;
    for (int i = threadIdx.x; i < K; i += 256) ss = fmaf(xr[i], xr[i], ss);
    ss = wave_sum(ss);
    if (lane == 63) red[wave] = ss;
    __syncthreads();
    inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)K + eps);
    __syncthreads();
  }
  float amax = 0.0f;
  for (int i = threadIdx.x; i < K; i += 256) {
    float v = xr[i];
    if (gain) v = gain[i] * (v * inv);
    amax = fmaxf(amax, fabsf(v));
  }
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  if (lane == 0) red[wave] = amax;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float a = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    int e = 0;
    if (a > 0.0f && a < 3.0e38f) { int ex; frexpf(a, &ex); e = 14 - ex; }   // a = m*2^ex, m in [0.5,1) -> a*2^e in [2^13, 2^14)
    if (e > 60) e = 60; if (e < -60) e = -60;
    s_scale = ldexpf(1.0f, e);
    sinv[t] = ldexpf(1.0f, -e);
  }
  __syncthreads();
  const float s = s_scale;
  // one 32-block per half-wave pass: 8 blocks per work-group pass
  const int hw = threadIdx.x >> 5, l32 = threadIdx.x & 31;
  for (int b = hw; b < (K >> 5); b += 8) {
    const int i = b * 32 + l32;
    float v = xr[i];
    if (gain) v = gain[i] * (v * inv);
    const float vs = v * s;
    const _Float16 h = (_Float16)vs;
    const _Float16 l = (_Float16)(vs - (float)h);
    hi[(int64_t)t * K + i] = h; lo[(int64_t)t * K + i] = l;
    float sum = v;
    for (int off = 16; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (l32 == 0) sx[(int64_t)t * (K >> 5) + b] = sum;
  }
}

struct GemmParams {
  const uint8_t* w; const float* bias;
  int rows, cols;
  const _Float16* xhi; const _Float16* xlo; const float* sx; const float* sinv;
  int n_tok;
  float* y; int64_t y_stride;       // y[t*y_stride + row]
  const float* residual;            // same indexing as y, may alias y
  int swiglu_half;                  // > 0: rows [0,half) up, [half,2half) gate; y[t*y_stride + i] = up*silu(gate)
};

__device__ __forceinline__ half4_t nib_to_half4(uint32_t t)
{
  // four integer bytes (0..15) -> four exact halfs: bytes become the low mantissa bits of 1024 + n, then -1024
  const uint32_t p01 = __builtin_amdgcn_perm(0x64646464u, t, 0x04010400u);
  const uint32_t p23 = __builtin_amdgcn_perm(0x64646464u, t, 0x04030402u);
  const half2_t k = {(_Float16)1024.0f, (_Float16)1024.0f};
  const half2_t a = __builtin_bit_cast(half2_t, p01) - k, b = __builtin_bit_cast(half2_t, p23) - k;
  return half4_t{a.x, a.y, b.x, b.y};
}

// One wave: 32 rows x 128 tokens.  MODE 0: plain rows (+bias, +residual).  MODE 1: SwiGLU pairs - the wave owns up rows
// R0..R0+31 AND the matching gate rows, two accumulator sets.
template <int MODE>
__global__ __launch_bounds__(256) void gemm_q4k_mfma(const GemmParams p)
{
  __shared__ __align__(16) _Float16 xs_hi[PF_TOK * PF_LDK];
  __shared__ __align__(16) _Float16 xs_lo[PF_TOK * PF_LDK];
  __shared__ __align__(16) float s_ab[4][(MODE == 1 ? 2 : 1)][4][32];   // [wave][matrix][a_lo,b_lo,a_hi,b_hi][row]
  constexpr int NM = MODE == 1 ? 2 : 1;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 31, kg = lane >> 5;
  const int n_out = MODE == 1 ? p.swiglu_half : p.rows;
  const int R0 = blockIdx.x * 128 + wave * 32;
  const int T0 = blockIdx.y * PF_TOK;
  const int K = p.cols, nsb = K >> 8;
  const int64_t row_bytes = (int64_t)nsb * 144;
  const uint8_t* wrow[NM];
#pragma unroll
  for (int mtx = 0; mtx < NM; mtx++) {
    int r = min(R0 + n, n_out - 1);
    if (MODE == 1 && mtx == 1) r += p.swiglu_half;
    wrow[mtx] = p.w + (int64_t)r * row_bytes;
  }
  float16_t Y[NM][4];
#pragma unroll
  for (int mtx = 0; mtx < NM; mtx++)
#pragma unroll
    for (int tt = 0; tt < 4; tt++)
#pragma unroll
      for (int v = 0; v < 16; v++) Y[mtx][tt][v] = 0.0f;
  float sinv_n[4];
#pragma unroll
  for (int tt = 0; tt < 4; tt++) { const int t = T0 + tt * 32 + n; sinv_n[tt] = t < p.n_tok ? p.sinv[t] : 0.0f; }

  uint4 hdr[NM];
  for (int k0 = 0; k0 < K; k0 += PF_KC) {
    const int sb = k0 >> 8, c = (k0 >> 6) & 3;
    // ---- stage the activation chunk: 128 tokens x 64 k (hi and lo) ----
    __syncthreads();
    {
      const int tok = threadIdx.x >> 1, half = threadIdx.x & 1;
      const int t = T0 + tok;
      uint4 h[4], l[4];
      if (t < p.n_tok) {
        const uint4* sh = reinterpret_cast<const uint4*>(p.xhi + (int64_t)t * K + k0 + half * 32);
        const uint4* sl = reinterpret_cast<const uint4*>(p.xlo + (int64_t)t * K + k0 + half * 32);
#pragma unroll
        for (int i = 0; i < 4; i++) { h[i] = sh[i]; l[i] = sl[i]; }
      } else {
#pragma unroll
        for (int i = 0; i < 4; i++) { h[i] = make_uint4(0, 0, 0, 0); l[i] = make_uint4(0, 0, 0, 0); }
      }
      // padded rows are only 8-byte aligned: store as 64-bit pieces
      uint2* dh = reinterpret_cast<uint2*>(xs_hi + tok * PF_LDK + half * 32);
      uint2* dl = reinterpret_cast<uint2*>(xs_lo + tok * PF_LDK + half * 32);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        dh[2 * i] = make_uint2(h[i].x, h[i].y); dh[2 * i + 1] = make_uint2(h[i].z, h[i].w);
        dl[2 * i] = make_uint2(l[i].x, l[i].y); dl[2 * i + 1] = make_uint2(l[i].z, l[i].w);
      }
    }
    // ---- weights of this chunk: 16 quant bytes per lane (elements 16kg .. 16kg+15 of both sub-blocks) ----
    half4_t A[NM][2][4];
#pragma unroll
    for (int mtx = 0; mtx < NM; mtx++) {
      const uint8_t* blk = wrow[mtx] + (int64_t)sb * 144;
      if (c == 0) hdr[mtx] = *reinterpret_cast<const uint4*>(blk);
      const uint4 q = *reinterpret_cast<const uint4*>(blk + 16 + 32 * c + 16 * kg);
      const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int m = 0; m < 4; m++) {
        A[mtx][0][m] = nib_to_half4(qw[m] & 0x0f0f0f0fu);
        A[mtx][1][m] = nib_to_half4((qw[m] >> 4) & 0x0f0f0f0fu);
      }
      if (kg == 0) {   // block scales of row n for sub-blocks 2c and 2c+1
        uint32_t sc, mn; q4k_scale_pair(hdr[mtx].y, hdr[mtx].z, hdr[mtx].w, c, sc, mn);
        const float d = __half2float(__ushort_as_half((unsigned short)(hdr[mtx].x & 0xffffu)));
        const float dmin = __half2float(__ushort_as_half((unsigned short)(hdr[mtx].x >> 16)));
        s_ab[wave][mtx][0][n] = d * cvt_ub0(sc); s_ab[wave][mtx][1][n] = dmin * cvt_ub0(mn);
        s_ab[wave][mtx][2][n] = d * cvt_ub1(sc); s_ab[wave][mtx][3][n] = dmin * cvt_ub1(mn);
      }
    }
    __syncthreads();

    // block sums of x for this lane's token column (two sub-blocks x four token tiles)
    float sxv[4][2];
#pragma unroll
    for (int tt = 0; tt < 4; tt++) {
      const int t = T0 + tt * 32 + n;
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) sxv[tt][s2] = t < p.n_tok ? p.sx[(int64_t)t * (K >> 5) + (k0 >> 5) + s2] : 0.0f;
    }
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++) {
      // per-row scales of this lane's 16 output rows: rows 8g + 4kg + (0..3)
      float av[NM][16], bv[NM][16];
#pragma unroll
      for (int mtx = 0; mtx < NM; mtx++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const float4 a4 = *reinterpret_cast<const float4*>(&s_ab[wave][mtx][2 * s2][8 * g + 4 * kg]);
          const float4 b4 = *reinterpret_cast<const float4*>(&s_ab[wave][mtx][2 * s2 + 1][8 * g + 4 * kg]);
          av[mtx][4 * g] = a4.x; av[mtx][4 * g + 1] = a4.y; av[mtx][4 * g + 2] = a4.z; av[mtx][4 * g + 3] = a4.w;
          bv[mtx][4 * g] = b4.x; bv[mtx][4 * g + 1] = b4.y; bv[mtx][4 * g + 2] = b4.z; bv[mtx][4 * g + 3] = b4.w;
        }
#pragma unroll
      for (int tt = 0; tt < 4; tt++) {
        const _Float16* bh = xs_hi + (tt * 32 + n) * PF_LDK + s2 * 32 + 16 * kg;
        const _Float16* bl = xs_lo + (tt * 32 + n) * PF_LDK + s2 * 32 + 16 * kg;
        half4_t Bh[4], Bl[4];
#pragma unroll
        for (int m = 0; m < 4; m++) { Bh[m] = *reinterpret_cast<const half4_t*>(bh + 4 * m); Bl[m] = *reinterpret_cast<const half4_t*>(bl + 4 * m); }
#pragma unroll
        for (int mtx = 0; mtx < NM; mtx++) {
          float16_t P;
#pragma unroll
          for (int v = 0; v < 16; v++) P[v] = 0.0f;
#pragma unroll
          for (int m = 0; m < 4; m++) {
            P = __builtin_amdgcn_mfma_f32_32x32x8f16(A[mtx][s2][m], Bh[m], P, 0, 0, 0);
            P = __builtin_amdgcn_mfma_f32_32x32x8f16(A[mtx][s2][m], Bl[m], P, 0, 0, 0);
          }
          const float si = sinv_n[tt], sxn = sxv[tt][s2];
#pragma unroll
          for (int v = 0; v < 16; v++) Y[mtx][tt][v] += (av[mtx][v] * si) * P[v] - bv[mtx][v] * sxn;
        }
      }
    }
  }

  // ---- write: lane holds column (token) n of each tile and rows 8g + 4kg + (0..3) ----
#pragma unroll
  for (int tt = 0; tt < 4; tt++) {
    const int t = T0 + tt * 32 + n;
    if (t >= p.n_tok) continue;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int row = R0 + 8 * (v >> 2) + 4 * kg + (v & 3);
      if (row >= n_out) continue;
      const int64_t o = (int64_t)t * p.y_stride + row;
      if (MODE == 0) {
        float r = Y[0][tt][v];
        if (p.bias) r += p.bias[row];
        if (p.residual) r += p.residual[o];
        p.y[o] = r;
      } else {
        float up = Y[0][tt][v], gate = Y[NM - 1][tt][v];
        if (p.bias) { up += p.bias[row]; gate += p.bias[p.swiglu_half + row]; }
        p.y[o] = silu_mul(up, gate);
      }
    }
  }
}

int launch_xprep(const float* x, int64_t x_stride, const float* gain, float eps, int K, int n_tok,
                 _Float16* hi, _Float16* lo, float* sx, float* sinv)
{
  hipLaunchKernelGGL(xprep_kernel, dim3(n_tok), dim3(256), 0, ctx().stream, x, x_stride, gain, eps, K, hi, lo, sx, sinv);
  return CAI_OK;
}

bool gemm_mfma_supported(const cai_qw_s* w) { return w->qtype == CAI_Q4_K; }

int launch_gemm_q4k(const cai_qw_s* w, const _Float16* xhi, const _Float16* xlo, const float* sx, const float* sinv,
                    int n_tok, float* y, int64_t y_stride, const float* residual, int swiglu_half)
{
  if (!gemm_mfma_supported(w)) return set_error(CAI_ERR_UNSUPPORTED, "prefill gemm: weight type %d", w->qtype);
  GemmParams p{};
  p.w = w->data; p.bias = w->bias; p.rows = (int)w->rows; p.cols = (int)w->cols;
  p.xhi = xhi; p.xlo = xlo; p.sx = sx; p.sinv = sinv; p.n_tok = n_tok; p.y = y; p.y_stride = y_stride;
  p.residual = residual; p.swiglu_half = swiglu_half;
  const int n_out = swiglu_half ? swiglu_half : p.rows;
  const dim3 grid((n_out + 127) / 128, (n_tok + PF_TOK - 1) / PF_TOK);
  if (swiglu_half) return set_error(CAI_ERR_UNSUPPORTED, "prefill gemm: fused SwiGLU is not built (two accumulator sets exceed the register file)");
  hipLaunchKernelGGL(gemm_q4k_mfma<0>, grid, dim3(256), 0, ctx().stream, p);
  return CAI_OK;
}

}  // namespace cai

// ------------------------------------------------------------------------------------------
// workspace + C ABI
// ------------------------------------------------------------------------------------------
namespace cai {
struct PrefillWs { _Float16* hi = nullptr; _Float16* lo = nullptr; float* sx = nullptr; float* sinv = nullptr; size_t cap_elems = 0; int cap_tok = 0; };
static PrefillWs g_pws;

int prefill_ws(int n_tok, int K, _Float16** hi, _Float16** lo, float** sx, float** sinv)
{
  const size_t need = (size_t)n_tok * K;
  if (need > g_pws.cap_elems || n_tok > g_pws.cap_tok) {
    CAI_HIP(hipStreamSynchronize(ctx().stream));
    if (g_pws.hi) { (void)hipFree(g_pws.hi); (void)hipFree(g_pws.lo); (void)hipFree(g_pws.sx); (void)hipFree(g_pws.sinv); g_pws = PrefillWs(); }
    const size_t ce = std::max(need, g_pws.cap_elems); const int ct = std::max(n_tok, g_pws.cap_tok);
    CAI_HIP(hipMalloc((void**)&g_pws.hi, ce * 2)); CAI_HIP(hipMalloc((void**)&g_pws.lo, ce * 2));
    CAI_HIP(hipMalloc((void**)&g_pws.sx, ce / 32 * 4 + 64)); CAI_HIP(hipMalloc((void**)&g_pws.sinv, (size_t)ct * 4));
    g_pws.cap_elems = ce; g_pws.cap_tok = ct;
  }
  *hi = g_pws.hi; *lo = g_pws.lo; *sx = g_pws.sx; *sinv = g_pws.sinv;
  return CAI_OK;
}

int prefill_prep(const float* x, int64_t x_stride, const float* gain, float eps, int K, int n_tok)
{
  _Float16 *hi, *lo; float *sx, *sinv; int rc;
  if ((rc = prefill_ws(n_tok, K, &hi, &lo, &sx, &sinv))) return rc;
  return launch_xprep(x, x_stride, gain, eps, K, n_tok, hi, lo, sx, sinv);
}
// Several matrices of one width applied to the prepared activations (q | k | v).
int prefill_gemm_multi(const cai_qw_s* const* ws, const int* y_off, int n_w, int n_tok, float* y, int64_t y_stride)
{
  for (int i = 0; i < n_w; i++) {
    const int rc = launch_gemm_q4k(ws[i], g_pws.hi, g_pws.lo, g_pws.sx, g_pws.sinv, n_tok, y + y_off[i], y_stride, nullptr, 0);
    if (rc) return rc;
  }
  return CAI_OK;
}
int prefill_gemm(const cai_qw_s* w, int n_tok, float* y, int64_t y_stride, const float* residual)
{
  return launch_gemm_q4k(w, g_pws.hi, g_pws.lo, g_pws.sx, g_pws.sinv, n_tok, y, y_stride, residual, 0);
}

// y[t][rows] = W x[t] (+bias) (+residual) for n_tok tokens; x rows are x_stride apart; gain != null fuses RMSNorm.
int prefill_linear(const cai_qw_s* w, const float* x, int64_t x_stride, const float* gain, float eps, int n_tok,
                   float* y, int64_t y_stride, const float* residual)
{
  int rc;
  if (gemm_mfma_supported(w) && n_tok <= 16) return nb_linear(w, x, x_stride, gain, eps, n_tok, y, y_stride, residual);   // bandwidth-bound regime
  if (gemm_mfma_supported(w)) {
    _Float16 *hi, *lo; float *sx, *sinv;
    if ((rc = prefill_ws(n_tok, (int)w->cols, &hi, &lo, &sx, &sinv))) return rc;
    launch_xprep(x, x_stride, gain, eps, (int)w->cols, n_tok, hi, lo, sx, sinv);
    return launch_gemm_q4k(w, hi, lo, sx, sinv, n_tok, y, y_stride, residual, 0);
  }
  // other weight types: groups of up to 8 tokens through the small-batch kernel (x must be contiguous)
  if (x_stride != w->cols) return set_error(CAI_ERR_UNSUPPORTED, "prefill linear: strided input needs a Q4_K matrix");
  for (int t = 0; t < n_tok; t += 8) {
    const int nb = std::min(8, n_tok - t);
    MultiGemv m{}; m.n = 1; m.w[0] = w; m.rows[0] = w->rows;
    if ((rc = launch_gemv_multi(m, x + (int64_t)t * w->cols, nb, y + (int64_t)t * y_stride, y_stride, CAI_ACT_NONE,
                                residual ? residual + (int64_t)t * y_stride : nullptr, gain, eps, 0))) return rc;
  }
  return CAI_OK;
}
}  // namespace cai

using namespace cai;

extern "C" int cai_qgemm(cai_qw_t w, const float* x, int n_tokens, float* y, int flags)
{
  CAI_READY();
  CAI_REQUIRE(w && x && y && n_tokens >= 1, "cai_qgemm: bad argument");
  Context& c = ctx();
  const size_t xb = (size_t)n_tokens * w->cols * 4, yb = (size_t)n_tokens * w->rows * 4;
  const float* dx = x; float* dy = y; int rc;
  if (!(flags & CAI_X_DEVICE)) {
    if ((rc = ensure_stage(&c.stage_in, &c.stage_in_cap, xb))) return rc;
    CAI_HIP(hipMemcpyAsync(c.stage_in, x, xb, hipMemcpyHostToDevice, c.stream));
    dx = (const float*)c.stage_in;
  }
  if (!(flags & CAI_Y_DEVICE)) { if ((rc = ensure_stage(&c.stage_out, &c.stage_out_cap, yb))) return rc; dy = (float*)c.stage_out; }
  if ((rc = prefill_linear(w, dx, w->cols, nullptr, 0.0f, n_tokens, dy, w->rows, nullptr))) return rc;
  CAI_HIP(hipGetLastError());
  if (!(flags & CAI_Y_DEVICE)) { CAI_HIP(hipMemcpyAsync(y, dy, yb, hipMemcpyDeviceToHost, c.stream)); CAI_HIP(hipStreamSynchronize(c.stream)); }
  return CAI_OK;
}
