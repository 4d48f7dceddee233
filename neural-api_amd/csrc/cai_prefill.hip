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


// ------------------------------------------------------------------------------------------
// Activation pre-pass (one work-group per token): optional RMSNorm (neural/neural.cl:1047-1085), then
//   s = 2^e with max|x|*s in [2^13, 2^14),  hi = f16(x*s),  lo = f16(x*s - hi),
//   sxhi[b] + sxlo[b] = (sum of x over 32-block b) * s / 32 as two halfs (the block sums go to the matrix cores too).
// SWIGLU: the row holds up | gate (K values each) and the value is up * silu(gate) - the feed-forward's middle step folded into
// the pre-pass of the down projection (no norm in that case).
// ------------------------------------------------------------------------------------------
template <bool SWIGLU, int NT>     // NT threads per token
__global__ __launch_bounds__(NT) void xprep_kernel(const float* x, int64_t x_stride, const float* gain, float eps, int K,
                                                    _Float16* hi, _Float16* lo, float* sinv, _Float16* sxhi, _Float16* sxlo)
{
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const float* xr = x + (int64_t)t * x_stride;
  __shared__ float red[NT / 64];
  __shared__ float s_scale;
  float inv = 1.0f;
  const float* second = SWIGLU ? xr + K : gain;     // the array walked beside x: the gate half, or the norm gain
  if (!SWIGLU && gain) {
    float ss = 0.0f;
    for_strided8(xr, threadIdx.x, K, NT, [&](float v, int) { ss = fmaf(v, v, ss); });
    ss = wave_sum(ss);
    if (lane == 63) red[wave] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int w4 = 0; w4 < NT / 64; w4 += 4) tot += (red[w4] + red[w4 + 1]) + (red[w4 + 2] + red[w4 + 3]);
    inv = 1.0f / sqrtf(tot / (float)K + eps);
    __syncthreads();
  }
  float amax = 0.0f;
  for_strided8(xr, second, threadIdx.x, K, NT, [&](float v, float g, int) {
    if (SWIGLU) v = silu_mul(v, g);
    else if (gain) v = g * (v * inv);
    amax = fmaxf(amax, fabsf(v));
  });
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  if (lane == 0) red[wave] = amax;
  __syncthreads();
  if (threadIdx.x == 0) {
    float a = 0.0f;
#pragma unroll
    for (int w4 = 0; w4 < NT / 64; w4++) a = fmaxf(a, red[w4]);
    int e = 0;
    if (a > 0.0f && a < 3.0e38f) { int ex; frexpf(a, &ex); e = 14 - ex; }   // a = m*2^ex, m in [0.5,1) -> a*2^e in [2^13, 2^14)
    if (e > 60) e = 60; if (e < -60) e = -60;
    s_scale = ldexpf(1.0f, e);
    sinv[t] = ldexpf(1.0f, -e);
  }
  __syncthreads();
  const float s = s_scale;
  // one 32-block per half-wave and turn (thread i of a turn takes element turn * 256 + i): 8 blocks per work-group turn
  for_strided8(xr, second, threadIdx.x, K, NT, [&](float v, float g, int i) {
    if (SWIGLU) v = silu_mul(v, g);
    else if (gain) v = g * (v * inv);
    const float vs = v * s;
    _Float16 h, l; split_f16(vs, h, l);
    hi[(int64_t)t * K + i] = h; lo[(int64_t)t * K + i] = l;
    float sum = v;
    for (int off = 16; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if ((i & 31) == 0) {   // the block sum in the scaled domain of hi/lo, divided by 32 so that it stays inside the half range
      const float ss = sum * s * 0.03125f;
      _Float16 sh, sl; split_f16(ss, sh, sl);
      sxhi[(int64_t)t * (K >> 5) + (i >> 5)] = sh; sxlo[(int64_t)t * (K >> 5) + (i >> 5)] = sl;
    }
  });
}

// The same pre-pass for rows of at most KE * NT values: every thread keeps its KE values in registers, so the row is read
// once (the general kernel above reads it for the sum of squares, for the maximum and for the conversion) and SwiGLU is
// evaluated once.  Thread i takes elements i, i + NT, ...: the order of every sum is that of the general kernel.
template <bool SWIGLU, int NT, int KE>
__global__ __launch_bounds__(NT) void xprep_regs_kernel(const float* x, int64_t x_stride, const float* gain, float eps, int K,
                                                         _Float16* hi, _Float16* lo, float* sinv, _Float16* sxhi, _Float16* sxlo)
{
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const float* xr = x + (int64_t)t * x_stride;
  const float* second = SWIGLU ? xr + K : gain;
  __shared__ float red[NT / 64];
  __shared__ float s_scale;
  float v[KE], g[KE];
#pragma unroll
  for (int e = 0; e < KE; e++) {                    // requests carry no branch: past the end the last value again (not used)
    const int j = min((int)threadIdx.x + e * NT, K - 1);
    v[e] = xr[j]; g[e] = second ? second[j] : 1.0f;
  }
  if (!SWIGLU && gain) {
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < KE; e++) if ((int)threadIdx.x + e * NT < K) ss = fmaf(v[e], v[e], ss);
    ss = wave_sum(ss);
    if (lane == 63) red[wave] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int w4 = 0; w4 < NT / 64; w4 += 4) tot += (red[w4] + red[w4 + 1]) + (red[w4 + 2] + red[w4 + 3]);
    const float inv = 1.0f / sqrtf(tot / (float)K + eps);
    __syncthreads();
#pragma unroll
    for (int e = 0; e < KE; e++) v[e] = g[e] * (v[e] * inv);
  } else if (SWIGLU) {
#pragma unroll
    for (int e = 0; e < KE; e++) v[e] = silu_mul(v[e], g[e]);
  }
  float amax = 0.0f;
#pragma unroll
  for (int e = 0; e < KE; e++) if ((int)threadIdx.x + e * NT < K) amax = fmaxf(amax, fabsf(v[e]));
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  if (lane == 0) red[wave] = amax;
  __syncthreads();
  if (threadIdx.x == 0) {
    float a = 0.0f;
#pragma unroll
    for (int w4 = 0; w4 < NT / 64; w4++) a = fmaxf(a, red[w4]);
    int ex2 = 0;
    if (a > 0.0f && a < 3.0e38f) { int ex; frexpf(a, &ex); ex2 = 14 - ex; }
    if (ex2 > 60) ex2 = 60; if (ex2 < -60) ex2 = -60;
    s_scale = ldexpf(1.0f, ex2);
    sinv[t] = ldexpf(1.0f, -ex2);
  }
  __syncthreads();
  const float s = s_scale;
#pragma unroll
  for (int e = 0; e < KE; e++) {
    const int i = (int)threadIdx.x + e * NT;
    if (i < K) {                                    // K is a multiple of 32: a half-wave is inside or outside together
      const float vs = v[e] * s;
      _Float16 h, l; split_f16(vs, h, l);
      hi[(int64_t)t * K + i] = h; lo[(int64_t)t * K + i] = l;
      float sum = v[e];
      for (int off = 16; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
      if ((i & 31) == 0) {
        const float ss = sum * s * 0.03125f;
        _Float16 sh, sl; split_f16(ss, sh, sl);
        sxhi[(int64_t)t * (K >> 5) + (i >> 5)] = sh; sxlo[(int64_t)t * (K >> 5) + (i >> 5)] = sl;
      }
    }
  }
}

template <bool SWIGLU>
static void xprep_launch(const float* x, int64_t x_stride, const float* gain, float eps, int K, int n_tok,
                         _Float16* hi, _Float16* lo, float* sinv, _Float16* sxhi, _Float16* sxlo)
{
  hipStream_t st = ctx().stream;
  if (K <= 16 * 256) hipLaunchKernelGGL((xprep_regs_kernel<SWIGLU, 256, 16>), dim3(n_tok), dim3(256), 0, st, x, x_stride, gain, eps, K, hi, lo, sinv, sxhi, sxlo);
  else if (K <= 24 * 1024) hipLaunchKernelGGL((xprep_regs_kernel<SWIGLU, 1024, 24>), dim3(n_tok), dim3(1024), 0, st, x, x_stride, gain, eps, K, hi, lo, sinv, sxhi, sxlo);
  else hipLaunchKernelGGL((xprep_kernel<SWIGLU, 1024>), dim3(n_tok), dim3(1024), 0, st, x, x_stride, gain, eps, K, hi, lo, sinv, sxhi, sxlo);
}

struct GemmParams {
  const uint8_t* w; const uint8_t* aux; const uint8_t* aux2; const float* bias;   // aux, aux2: Q6_K planes of scales and of d
  int rows, cols;
  const _Float16* xhi; const _Float16* xlo;     // [token][cols]
  const _Float16* sxhi; const _Float16* sxlo;   // [token][cols/32]
  const float* sinv;                            // [token]
  int n_tok;
  float* y; int64_t y_stride;       // y[t*y_stride + row]
  const float* residual;            // same indexing as y, may alias y
  int n_row_groups, n_tok_tiles;
  // up to two more matrices of the same type and width in the same launch (q | k | v): row groups [seg_end[i], ...) belong to
  // matrix i + 1, whose rows land y_off2[i] columns into a y row (gemm_q4k_pf only)
  int n_seg; int seg_end[2];
  const uint8_t* w2[2]; const float* bias2[2]; int rows2[2]; int y_off2[2];
  // fused feed-forward front half (gemm_q4k_pf with two row tiles per wave): rows [0, half) are up, [half, 2 half) gate; a wave's
  // two tiles are 32 up rows and THEIR gate rows, and y[t][i] = up_i * silu(gate_i) is written (y rows are half wide)
  int swiglu_half;
};

constexpr int PF_LDX = 264;       // halfs per staged token row: 256 + pad (stride = 4 banks mod 64: 16-byte reads)

__device__ __forceinline__ half4_t bytes_to_half4_pf(uint32_t t)
{
  // four bytes (0..255) -> four exact halfs 1024 + b (the byte becomes the low mantissa bits of 0x6400 = 1024.0)
  const uint32_t p01 = __builtin_amdgcn_perm(0x64646464u, t, 0x04010400u);
  const uint32_t p23 = __builtin_amdgcn_perm(0x64646464u, t, 0x04030402u);
  const half2_t a = __builtin_bit_cast(half2_t, p01), b = __builtin_bit_cast(half2_t, p23);
  return half4_t{a.x, a.y, b.x, b.y};
}

typedef _Float16 half8_pf __attribute__((ext_vector_type(8)));

// One work-group: 4 waves x RT row tiles of 32 rows x TT * 32 tokens, one super-block (256 columns) per step, on
// v_mfma_f32_32x32x16_f16 (lane (n, kg) supplies 8 consecutive k of row / column n).
//   * the weight operand sc_j * q (<= 63 * 15, exact in f16) is built once per super-block per wave and reused by the
//     token tiles and by the hi and lo activation planes; the matrix cores accumulate across the whole super-block, hi
//     and lo planes into the same accumulator (the chains of the tiles interleave);
//   * -dmin * mn_j * sum_{k in j} x_k is one more MFMA step per plane (k = the 8 sub-blocks);
//   * d and dmin are applied once per super-block (2 FMAs per value), the token scale once at the end.
// Every MFMA takes its activation operand from LDS (1 KB per wave and instruction): with one row tile per wave the LDS
// pipe, not the matrix cores, sets the pace.  RT = 2 lets one activation operand serve two row tiles (half the LDS reads
// per FLOP); it needs 256 rows per work-group and is used for matrices with enough row groups to fill the chip.
// Work-group ids are laid out so that the token tiles of one row group run on one XCD: the re-reads of its weights (one
// per token tile) hit that XCD's L2.  TT = 1 doubles the number of work-groups for matrices with few row groups.
// QT = CAI_Q5_K: 176-byte super-blocks (neural/neuralgguf.pas:516-587) - the Q4_K header, the 32-byte plane of fifth bits (bit j of byte i
// belongs to weight i of sub-block j), the nibbles; the weight operand sc * (nibble | bit << 4) <= 63 * 31 stays exact in f16.
template <int TT, int RT, int QT>
__global__ __launch_bounds__(256, 2) void gemm_q4k_pf(const GemmParams p)
{
  constexpr int BB = QT == CAI_Q5_K ? 176 : 144, QOFF = QT == CAI_Q5_K ? 48 : 16;
  extern __shared__ __align__(16) unsigned char pf_smem[];
  constexpr int NTOK = TT * 32;
  _Float16* xs_hi = reinterpret_cast<_Float16*>(pf_smem);            // [NTOK][PF_LDX]
  _Float16* xs_lo = xs_hi + NTOK * PF_LDX;
  _Float16* sx_hi = xs_lo + NTOK * PF_LDX;                            // [NTOK][8]
  _Float16* sx_lo = sx_hi + NTOK * 8;
  float* s_d = reinterpret_cast<float*>(sx_lo + NTOK * 8);            // [4 waves][RT][2][32]
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, kg = lane >> 5;
  // linear id = rg_lo + 8 * (tt + n_tok_tiles * rg_hi): a row group's token tiles share id mod 8
  const int L = blockIdx.x, rg = (L & 7) + 8 * ((L >> 3) / p.n_tok_tiles), ttile = (L >> 3) % p.n_tok_tiles;
  if (rg >= p.n_row_groups) return;
  const uint8_t* wbase = p.w; const float* bias = p.bias; int rows = p.rows, yo = 0, rgl = rg;   // this work-group's matrix (uniform)
  if (p.n_seg > 1 && rg >= p.seg_end[0]) { wbase = p.w2[0]; bias = p.bias2[0]; rows = p.rows2[0]; yo = p.y_off2[0]; rgl = rg - p.seg_end[0]; }
  if (p.n_seg > 2 && rg >= p.seg_end[1]) { wbase = p.w2[1]; bias = p.bias2[1]; rows = p.rows2[1]; yo = p.y_off2[1]; rgl = rg - p.seg_end[1]; }
  const int half = RT == 2 ? p.swiglu_half : 0;
  const int R0 = half ? (rgl * 4 + wave) * 32 : (rgl * 4 + wave) * 32 * RT, T0 = ttile * NTOK;
  const int K = p.cols, nsb = K >> 8, nb32 = K >> 5;
  const int64_t row_bytes = (int64_t)nsb * BB;
  const uint8_t* wrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++) {     // tail rows: re-read the last row, not written
    const int row = half ? min(R0 + n, half - 1) + rt * half : min(R0 + 32 * rt + n, rows - 1);
    wrow[rt] = wbase + (int64_t)row * row_bytes;
  }

  struct WRegs { uint4 h, q[4], e[QT == CAI_Q5_K ? 2 : 1]; };   // e: Q5_K's bit plane (all 32 bytes: the lane needs four bits of each)
  auto load_w = [&](int sb, WRegs (&r)[RT]) {
    if (sb < nsb) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        const uint8_t* blk = wrow[rt] + (int64_t)sb * BB;
        r[rt].h = *reinterpret_cast<const uint4*>(blk);
        if constexpr (QT == CAI_Q5_K) { r[rt].e[0] = *reinterpret_cast<const uint4*>(blk + 16); r[rt].e[1] = *reinterpret_cast<const uint4*>(blk + 32); }
#pragma unroll
        for (int i = 0; i < 4; i++) r[rt].q[i] = *reinterpret_cast<const uint4*>(blk + QOFF + 64 * kg + 16 * i);
      }
    }
  };
  float16_t Y[RT][TT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++)
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
      for (int v = 0; v < 16; v++) Y[rt][tt][v] = 0.0f;

  WRegs wcur[RT], wnxt[RT];
  load_w(0, wcur);
  for (int sb = 0; sb < nsb; sb++) {
    __syncthreads();                       // the previous step's LDS reads are done
    // ---- stage NTOK tokens x 256 columns of both planes, and the block sums ----
    {
      // thread = (token tq + 8 i, 16-byte chunk): offsets from the uniform plane pointers stay 32-bit.  Token rows past
      // the end repeat the last token (their results are never written), so the loads carry no branch and issue together.
      const int tq = threadIdx.x >> 5, chunk = threadIdx.x & 31;
      const uint32_t colo = (uint32_t)(sb * 256 + chunk * 8);
      constexpr int SB = (TT == 2 || RT == 2) ? 1 : 4;     // loads in flight per plane (measured: with two tiles the registers are worth more than the overlap)
#pragma unroll
      for (int i0 = 0; i0 < NTOK / 8; i0 += SB) {
        uint4 vh[SB], vl[SB];
#pragma unroll
        for (int i = 0; i < SB; i++) {
          const uint32_t off = (uint32_t)min(T0 + tq + 8 * (i0 + i), p.n_tok - 1) * (uint32_t)K + colo;
          vh[i] = *reinterpret_cast<const uint4*>(p.xhi + off);
          vl[i] = *reinterpret_cast<const uint4*>(p.xlo + off);
        }
#pragma unroll
        for (int i = 0; i < SB; i++) {
          *reinterpret_cast<uint4*>(xs_hi + (tq + 8 * (i0 + i)) * PF_LDX + chunk * 8) = vh[i];
          *reinterpret_cast<uint4*>(xs_lo + (tq + 8 * (i0 + i)) * PF_LDX + chunk * 8) = vl[i];
        }
      }
    }
    if (threadIdx.x < NTOK * 2) {
      const int tok = threadIdx.x % NTOK, plane = threadIdx.x / NTOK;
      const uint4 v = *reinterpret_cast<const uint4*>((plane ? p.sxlo : p.sxhi) + (int64_t)min(T0 + tok, p.n_tok - 1) * nb32 + sb * 8);
      *reinterpret_cast<uint4*>((plane ? sx_lo : sx_hi) + tok * 8) = v;
    }
    load_w(sb + 1, wnxt);
    __syncthreads();

    // ---- weight operand of this super-block: per row tile 16 groups of eight sc*q values ----
    const _Float16 k1024 = (_Float16)1024.0f;
    half8_pf A[RT][4][4];
    half4_t mnv[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
      const WRegs& r = wcur[rt];
      const uint32_t sc4 = kg == 0 ? (r.h.y & 0x3f3f3f3fu) : ((r.h.w & 0x0f0f0f0fu) | ((r.h.y >> 2) & 0x30303030u));
      const uint32_t mn4 = kg == 0 ? (r.h.z & 0x3f3f3f3fu) : (((r.h.w >> 4) & 0x0f0f0f0fu) | ((r.h.z >> 2) & 0x30303030u));
      const half4_t sch = bytes_to_half4_pf(sc4), mnh = bytes_to_half4_pf(mn4);
      const half4_t scv = half4_t{sch.x - k1024, sch.y - k1024, sch.z - k1024, sch.w - k1024};
      mnv[rt] = half4_t{mnh.x - k1024, mnh.y - k1024, mnh.z - k1024, mnh.w - k1024};
      if (kg == 0) {
        const float d = __half2float(__ushort_as_half((unsigned short)(r.h.x & 0xffffu)));
        const float dmin = __half2float(__ushort_as_half((unsigned short)(r.h.x >> 16)));
        s_d[((wave * RT + rt) * 2 + 0) * 32 + n] = d; s_d[((wave * RT + rt) * 2 + 1) * 32 + n] = dmin * 32.0f;
      }
#pragma unroll
      for (int j = 0; j < 4; j++) {                                      // sub-block 4kg + j: bytes of chunk 2kg + (j >> 1), low or high nibbles
        const int ccl = j >> 1, hl = j & 1;
        const _Float16 sj = j == 0 ? scv.x : (j == 1 ? scv.y : (j == 2 ? scv.z : scv.w));
        const half2_t s2 = {sj, sj};
        const half2_t c2 = {(_Float16)(-1024.0f) * sj, (_Float16)(-1024.0f) * sj};   // exact: a multiple of 1024 below 65504
#pragma unroll
        for (int t = 0; t < 4; t++) {                                    // weights 8t .. 8t+7 of the sub-block
          const uint4& qq = r.q[2 * ccl + (t >> 1)];
          const uint32_t qa = (t & 1) ? qq.z : qq.x, qb = (t & 1) ? qq.w : qq.y;
          uint32_t na = hl ? ((qa >> 4) & 0x0f0f0f0fu) : (qa & 0x0f0f0f0fu);
          uint32_t nb = hl ? ((qb >> 4) & 0x0f0f0f0fu) : (qb & 0x0f0f0f0fu);
          if constexpr (QT == CAI_Q5_K) {   // plane bytes 8 t .. 8 t + 7, bit 4 kg + j
            const uint4& ee = r.e[t >> 1];
            const uint32_t e0 = (t & 1) ? ee.z : ee.x, e1 = (t & 1) ? ee.w : ee.y;
            na |= ((e0 >> (4 * kg + j)) & 0x01010101u) << 4; nb |= ((e1 >> (4 * kg + j)) & 0x01010101u) << 4;
          }
          const half2_t a0 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, na, 0x04010400u)), s2, c2);   // (1024 + q) * sc - 1024 * sc = sc * q
          const half2_t a1 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, na, 0x04030402u)), s2, c2);
          const half2_t a2 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, nb, 0x04010400u)), s2, c2);
          const half2_t a3 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, nb, 0x04030402u)), s2, c2);
          A[rt][j][t] = half8_pf{a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
        }
      }
    }
    float16_t C[RT][TT], Cm[RT][TT];
    const float16_t zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int t = 0; t < 4; t++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
          const int off = (tt * 32 + n) * PF_LDX + 128 * kg + 32 * j + 8 * t;
          const half8_pf Bh = *reinterpret_cast<const half8_pf*>(xs_hi + off);
          const half8_pf Bl = *reinterpret_cast<const half8_pf*>(xs_lo + off);
#pragma unroll
          for (int rt = 0; rt < RT; rt++) {
            if (j == 0 && t == 0) C[rt][tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[rt][j][t], Bh, zero16, 0, 0, 0);   // a fresh accumulator per super-block
            else C[rt][tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[rt][j][t], Bh, C[rt][tt], 0, 0, 0);
          }
#pragma unroll
          for (int rt = 0; rt < RT; rt++) C[rt][tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[rt][j][t], Bl, C[rt][tt], 0, 0, 0);
        }
    __builtin_amdgcn_wave_barrier();       // s_d was written by this wave's own lanes above; LDS operations of a wave complete in order
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
      const half4_t Bmh = *reinterpret_cast<const half4_t*>(sx_hi + (tt * 32 + n) * 8 + 4 * kg);
      const half4_t Bml = *reinterpret_cast<const half4_t*>(sx_lo + (tt * 32 + n) * 8 + 4 * kg);
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        Cm[rt][tt] = __builtin_amdgcn_mfma_f32_32x32x8f16(mnv[rt], Bmh, zero16, 0, 0, 0);
        Cm[rt][tt] = __builtin_amdgcn_mfma_f32_32x32x8f16(mnv[rt], Bml, Cm[rt][tt], 0, 0, 0);
      }
#pragma unroll
      for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const float4 d4 = *reinterpret_cast<const float4*>(&s_d[((wave * RT + rt) * 2 + 0) * 32 + 8 * g + 4 * kg]);
          const float4 m4 = *reinterpret_cast<const float4*>(&s_d[((wave * RT + rt) * 2 + 1) * 32 + 8 * g + 4 * kg]);
          Y[rt][tt][4 * g + 0] += d4.x * C[rt][tt][4 * g + 0] - m4.x * Cm[rt][tt][4 * g + 0];
          Y[rt][tt][4 * g + 1] += d4.y * C[rt][tt][4 * g + 1] - m4.y * Cm[rt][tt][4 * g + 1];
          Y[rt][tt][4 * g + 2] += d4.z * C[rt][tt][4 * g + 2] - m4.z * Cm[rt][tt][4 * g + 2];
          Y[rt][tt][4 * g + 3] += d4.w * C[rt][tt][4 * g + 3] - m4.w * Cm[rt][tt][4 * g + 3];
        }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int rt = 0; rt < RT; rt++) wcur[rt] = wnxt[rt];
  }

  // ---- write: lane holds column (token) n of each tile and rows 8g + 4kg + (0..3): four consecutive outputs of a token
  // row go out as one 16-byte store (bias and residual come in the same way) when the addresses allow it ----
  const bool vec = ((p.y_stride | yo) & 3) == 0 && (reinterpret_cast<uintptr_t>(p.y) & 15) == 0 &&
                   (!p.residual || (reinterpret_cast<uintptr_t>(p.residual) & 15) == 0) && (!bias || (reinterpret_cast<uintptr_t>(bias) & 15) == 0);
  if constexpr (RT == 2) if (half) {
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
      const int t = T0 + tt * 32 + n;
      if (t >= p.n_tok) continue;
      const float si = p.sinv[t];
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int row = R0 + 8 * g + 4 * kg;
        const int64_t o = (int64_t)t * p.y_stride + row;
        float r[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float up = Y[0][tt][4 * g + i] * si, gate = Y[1][tt][4 * g + i] * si;
          if (bias && row + i < half) { up += bias[row + i]; gate += bias[half + row + i]; }
          r[i] = silu_mul(up, gate);
        }
        if (vec && row + 3 < half) *reinterpret_cast<float4*>(p.y + o) = make_float4(r[0], r[1], r[2], r[3]);
        else {
#pragma unroll
          for (int i = 0; i < 4; i++) if (row + i < half) p.y[o + i] = r[i];
        }
      }
    }
    return;
  }
#pragma unroll
  for (int tt = 0; tt < TT; tt++) {
    const int t = T0 + tt * 32 + n;
    if (t >= p.n_tok) continue;
    const float si = p.sinv[t];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int row = R0 + 32 * rt + 8 * g + 4 * kg;
        const int64_t o = (int64_t)t * p.y_stride + yo + row;
        if (vec && row + 3 < rows) {
          float4 r = make_float4(Y[rt][tt][4 * g] * si, Y[rt][tt][4 * g + 1] * si, Y[rt][tt][4 * g + 2] * si, Y[rt][tt][4 * g + 3] * si);
          if (bias) { const float4 b = *reinterpret_cast<const float4*>(bias + row); r.x += b.x; r.y += b.y; r.z += b.z; r.w += b.w; }
          if (p.residual) { const float4 q = *reinterpret_cast<const float4*>(p.residual + o); r.x += q.x; r.y += q.y; r.z += q.z; r.w += q.w; }
          *reinterpret_cast<float4*>(p.y + o) = r;
        } else {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            if (row + i >= rows) continue;
            float r = Y[rt][tt][4 * g + i] * si;
            if (bias) r += bias[row + i];
            if (p.residual) r += p.residual[o + i];
            p.y[o + i] = r;
          }
        }
      }
  }
}

// ------------------------------------------------------------------------------------------
// Q6_K on the same tiles (128 rows x TT * 32 tokens per work-group; neural/neuralgguf.pas:639-717).  A weight is
// d * scale * (q - 32) with one signed 8-bit scale per 16 weights, and scale * (q - 32) reaches 4096: not exact in f16.
// The scale is split, scale = 16 * (scale >> 4) + (scale & 15), and each weight takes TWO of the k slots of an MFMA:
// (q - 32) * 16 * (scale >> 4) (a multiple of 16 up to 4096) and (q - 32) * (scale & 15) (at most 480) are both exact,
// and the activation operand simply holds every value twice.  A lane (row n, half kg of the super-block) owns the 128
// weights of its half; a step of the chain covers the 4 weights 32 j + l4 .. + 3 of the half: one dword of ql (nibble
// j >> 1), one of qh (2-bit field j), the scale of group 2 j + (l4 >> 4).  There is no minimum term; d is applied once
// per super-block.  Resident form: 192-byte ql | qh records, a plane of scales, a plane of d.
// ------------------------------------------------------------------------------------------
template <int TT>
__global__ __launch_bounds__(256, 2) void gemm_q6k_pf(const GemmParams p)
{
  extern __shared__ __align__(16) unsigned char pf_smem[];
  constexpr int NTOK = TT * 32;
  _Float16* xs_hi = reinterpret_cast<_Float16*>(pf_smem);            // [NTOK][PF_LDX]
  _Float16* xs_lo = xs_hi + NTOK * PF_LDX;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, kg = lane >> 5;
  const int L = blockIdx.x, rg = (L & 7) + 8 * ((L >> 3) / p.n_tok_tiles), ttile = (L >> 3) % p.n_tok_tiles;
  if (rg >= p.n_row_groups) return;
  const int R0 = (rg * 4 + wave) * 32, T0 = ttile * NTOK;
  const int K = p.cols, nsb = K >> 8;
  const int64_t blk0 = (int64_t)min(R0 + n, p.rows - 1) * nsb;       // tail rows: re-read the last row, not written

  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
  struct WRegs { u32x4_t ql[4], qh[2]; u32x2_t sc; uint32_t d; };
  auto load_w = [&](int sb, WRegs& r) {          // unconditional: past the last super-block the last one is fetched again
    const int64_t b = blk0 + min(sb, nsb - 1);
    const uint8_t* rec = p.w + b * 192;
#pragma unroll
    for (int i = 0; i < 4; i++) r.ql[i] = *reinterpret_cast<const u32x4_t*>(rec + 64 * kg + 16 * i);
#pragma unroll
    for (int i = 0; i < 2; i++) r.qh[i] = *reinterpret_cast<const u32x4_t*>(rec + 128 + 32 * kg + 16 * i);
    r.sc = *reinterpret_cast<const u32x2_t*>(p.aux + b * 16 + 8 * kg);
    r.d = *reinterpret_cast<const uint16_t*>(p.aux2 + b * 2);
  };
  float16_t Y[TT];
#pragma unroll
  for (int tt = 0; tt < TT; tt++)
#pragma unroll
    for (int v = 0; v < 16; v++) Y[tt][v] = 0.0f;

  WRegs wcur, wnxt;
  load_w(0, wcur);
  for (int sb = 0; sb < nsb; sb++) {
    __syncthreads();                       // the previous step's LDS reads are done
    {
      const int tq = threadIdx.x >> 5, chunk = threadIdx.x & 31;
      const uint32_t colo = (uint32_t)(sb * 256 + chunk * 8);
      constexpr int SB = TT == 2 ? 1 : 4;
#pragma unroll
      for (int i0 = 0; i0 < NTOK / 8; i0 += SB) {
        uint4 vh[SB], vl[SB];
#pragma unroll
        for (int i = 0; i < SB; i++) {
          const uint32_t off = (uint32_t)min(T0 + tq + 8 * (i0 + i), p.n_tok - 1) * (uint32_t)K + colo;
          vh[i] = *reinterpret_cast<const uint4*>(p.xhi + off);
          vl[i] = *reinterpret_cast<const uint4*>(p.xlo + off);
        }
#pragma unroll
        for (int i = 0; i < SB; i++) {
          *reinterpret_cast<uint4*>(xs_hi + (tq + 8 * (i0 + i)) * PF_LDX + chunk * 8) = vh[i];
          *reinterpret_cast<uint4*>(xs_lo + (tq + 8 * (i0 + i)) * PF_LDX + chunk * 8) = vl[i];
        }
      }
    }
    load_w(sb + 1, wnxt);
    __syncthreads();

    const WRegs& r = wcur;
    // the 8 scales of this half as exact halfs: 16 * (s >> 4) (from the byte's top nibble, sign kept) and s & 15
    const uint32_t scw[2] = {r.sc.x, r.sc.y};
    half2_t s_hi[8], s_lo[8];
#pragma unroll
    for (int g = 0; g < 8; g++) {
      const int sc = (int)(int8_t)((scw[g >> 2] >> (8 * (g & 3))) & 0xffu);
      const _Float16 h = (_Float16)(float)((sc >> 4) * 16), l = (_Float16)(float)(sc & 15);
      s_hi[g] = half2_t{h, h}; s_lo[g] = half2_t{l, l};
    }
    const half2_t o2 = {(_Float16)(-1056.0f), (_Float16)(-1056.0f)};   // 1024 + q - 1056 = q - 32
    float16_t C[TT];
    const float16_t zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int w = 0; w < 8; w++) {                                      // l4 = 4 w
        const u32x4_t qlv = r.ql[2 * (j & 1) + (w >> 2)], qhv = r.qh[w >> 2];
        const uint32_t ql = qlv[w & 3], qh = qhv[w & 3];
        const uint32_t lo = (j >> 1) ? ((ql >> 4) & 0x0f0f0f0fu) : (ql & 0x0f0f0f0fu);
        const uint32_t hi = (j == 0 ? (qh << 4) : j == 1 ? (qh << 2) : j == 2 ? qh : (qh >> 2)) & 0x30303030u;
        const uint32_t c = lo | hi;
        const half2_t c01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, c, 0x04010400u)) + o2;
        const half2_t c23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, c, 0x04030402u)) + o2;
        const int g = 2 * j + (w >> 2);
        const half2_t a0 = c01 * s_hi[g], a1 = c23 * s_hi[g], a2 = c01 * s_lo[g], a3 = c23 * s_lo[g];
        const half8_pf A = {a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
          const int off = (tt * 32 + n) * PF_LDX + 128 * kg + 32 * j + 4 * w;
          const half4_t xh = *reinterpret_cast<const half4_t*>(xs_hi + off);
          const half4_t xl = *reinterpret_cast<const half4_t*>(xs_lo + off);
          const half8_pf Bh = {xh.x, xh.y, xh.z, xh.w, xh.x, xh.y, xh.z, xh.w};
          const half8_pf Bl = {xl.x, xl.y, xl.z, xl.w, xl.x, xl.y, xl.z, xl.w};
          if (j == 0 && w == 0) C[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A, Bh, zero16, 0, 0, 0);
          else C[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A, Bh, C[tt], 0, 0, 0);
          C[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A, Bl, C[tt], 0, 0, 0);
        }
      }
    // d of result row 8 g + 4 kg + i: held by the lane whose n is that row (both kg copies carry it)
    const float dmine = __half2float(__ushort_as_half((unsigned short)r.d));
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const float dv = __shfl(dmine, 8 * (v >> 2) + 4 * kg + (v & 3), 64);
#pragma unroll
      for (int tt = 0; tt < TT; tt++) Y[tt][v] = fmaf(dv, C[tt][v], Y[tt][v]);
    }
    wcur = wnxt;
  }

  const bool vec = (p.y_stride & 3) == 0 && (reinterpret_cast<uintptr_t>(p.y) & 15) == 0 &&
                   (!p.residual || (reinterpret_cast<uintptr_t>(p.residual) & 15) == 0) && (!p.bias || (reinterpret_cast<uintptr_t>(p.bias) & 15) == 0);
#pragma unroll
  for (int tt = 0; tt < TT; tt++) {
    const int t = T0 + tt * 32 + n;
    if (t >= p.n_tok) continue;
    const float si = p.sinv[t];
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const int row = R0 + 8 * g + 4 * kg;
      const int64_t o = (int64_t)t * p.y_stride + row;
      if (vec && row + 3 < p.rows) {
        float4 r = make_float4(Y[tt][4 * g] * si, Y[tt][4 * g + 1] * si, Y[tt][4 * g + 2] * si, Y[tt][4 * g + 3] * si);
        if (p.bias) { const float4 b = *reinterpret_cast<const float4*>(p.bias + row); r.x += b.x; r.y += b.y; r.z += b.z; r.w += b.w; }
        if (p.residual) { const float4 q = *reinterpret_cast<const float4*>(p.residual + o); r.x += q.x; r.y += q.y; r.z += q.z; r.w += q.w; }
        *reinterpret_cast<float4*>(p.y + o) = r;
      } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          if (row + i >= p.rows) continue;
          float r = Y[tt][4 * g + i] * si;
          if (p.bias) r += p.bias[row + i];
          if (p.residual) r += p.residual[o + i];
          p.y[o + i] = r;
        }
      }
    }
  }
}

int launch_xprep(const float* x, int64_t x_stride, const float* gain, float eps, int K, int n_tok,
                 _Float16* hi, _Float16* lo, float* sinv, _Float16* sxhi, _Float16* sxlo)
{
  xprep_launch<false>(x, x_stride, gain, eps, K, n_tok, hi, lo, sinv, sxhi, sxlo);
  return CAI_OK;
}

bool gemm_mfma_supported(const cai_qw_s* w) { return (w->qtype == CAI_Q4_K || w->qtype == CAI_Q5_K || w->qtype == CAI_Q6_K) && w->cols % 256 == 0; }

int launch_gemm_q4k(const cai_qw_s* w, const _Float16* xhi, const _Float16* xlo, const _Float16* sxhi, const _Float16* sxlo, const float* sinv,
                    int n_tok, float* y, int64_t y_stride, const float* residual)
{
  const int zero = 0;
  return launch_gemm_q4k_multi(&w, &zero, 1, xhi, xlo, sxhi, sxlo, sinv, n_tok, y, y_stride, residual, 0);
}

// Matrices of one type and width that one launch of the Q4_K / Q5_K prompt kernel can take together
bool gemm_q4k_multi_supported(const cai_qw_s* const* ws, int n_w)
{
  if (n_w < 1 || n_w > 3 || !gemm_mfma_supported(ws[0]) || ws[0]->qtype == CAI_Q6_K) return false;
  for (int i = 1; i < n_w; i++) if (ws[i]->qtype != ws[0]->qtype || ws[i]->cols != ws[0]->cols) return false;
  return true;
}

// y[t][y_off[i] + r] = (W_i x[t])[r] (+ bias_i) for up to three matrices of one type and width; one matrix: y_off[0] = 0, residual allowed.
// swiglu_half != 0 (one matrix of 2 * swiglu_half rows, no residual): y[t][i] = up_i * silu(gate_i), y rows swiglu_half wide.
int launch_gemm_q4k_multi(const cai_qw_s* const* ws, const int* y_off, int n_w, const _Float16* xhi, const _Float16* xlo, const _Float16* sxhi,
                          const _Float16* sxlo, const float* sinv, int n_tok, float* y, int64_t y_stride, const float* residual, int swiglu_half)
{
  const cai_qw_s* w = ws[0];
  if (!gemm_mfma_supported(w)) return set_error(CAI_ERR_UNSUPPORTED, "prefill gemm: weight type %d", w->qtype);
  if (n_w > 1 && (!gemm_q4k_multi_supported(ws, n_w) || residual)) return set_error(CAI_ERR_UNSUPPORTED, "prefill gemm: %d matrices in one launch", n_w);
  if (swiglu_half && (n_w != 1 || residual || w->qtype == CAI_Q6_K || w->rows != 2 * (int64_t)swiglu_half))
    return set_error(CAI_ERR_UNSUPPORTED, "prefill gemm: fused SwiGLU needs one Q4_K / Q5_K matrix of 2 x %d rows", swiglu_half);
  GemmParams p{};
  p.w = w->data; p.bias = w->bias; p.rows = (int)w->rows; p.cols = (int)w->cols;
  p.xhi = xhi; p.xlo = xlo; p.sxhi = sxhi; p.sxlo = sxlo; p.sinv = sinv; p.n_tok = n_tok; p.y = y + y_off[0]; p.y_stride = y_stride;
  p.residual = residual; p.n_seg = n_w;
  int64_t rows_all = 0;
  for (int i = 0; i < n_w; i++) rows_all += ws[i]->rows;
  if (w->qtype == CAI_Q6_K) {
    p.aux = w->aux; p.aux2 = qw_aux2(w);
    const int tt = ((p.rows + 127) / 128) * ((n_tok + 63) / 64) < 2 * ctx().n_cu ? 1 : 2;
    p.n_row_groups = (p.rows + 127) / 128;
    p.n_tok_tiles = (n_tok + tt * 32 - 1) / (tt * 32);
    const size_t lds = (size_t)tt * 32 * PF_LDX * 2 * 2;
    static bool attr6 = false;
    if (!attr6) {
      const void* ks[2] = {(const void*)gemm_q6k_pf<1>, (const void*)gemm_q6k_pf<2>};
      for (const void* k : ks) if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess) (void)hipGetLastError();
      attr6 = true;
    }
    const int grid = 8 * p.n_tok_tiles * ((p.n_row_groups + 7) / 8);
    if (tt == 1) hipLaunchKernelGGL(gemm_q6k_pf<1>, dim3(grid), dim3(256), lds, ctx().stream, p);
    else hipLaunchKernelGGL(gemm_q6k_pf<2>, dim3(grid), dim3(256), lds, ctx().stream, p);
    return CAI_OK;
  }
  // Tiling: two row tiles per wave (256 rows per work-group, 32 tokens) when that still gives every CU several
  // work-groups; else 128 rows with two token tiles, or with one for matrices with few row groups.
  const int n_cu = ctx().n_cu;
  const int wgs_rt2 = (int)((rows_all + 255) / 256) * ((n_tok + 31) / 32);
  const int wgs_tt2 = (int)((rows_all + 127) / 128) * ((n_tok + 63) / 64);
  // (measured on 512-token chunks: 7168 rows = 448 work-groups of two row tiles 107 us against 121 us with one tile; 5120 rows = 320
  // work-groups lose to 640 of one tile, 3584 rows = 224 likewise)
  const int mode = (swiglu_half || 4 * wgs_rt2 >= 7 * n_cu) ? 3 : (wgs_tt2 < 2 * n_cu ? 1 : 2);   // 1, 2: token tiles; 3: two row tiles
  const int rt = mode == 3 ? 2 : 1, tt = mode == 2 ? 2 : 1;
  p.swiglu_half = swiglu_half;
  p.n_row_groups = 0;
  for (int i = 0; i < n_w; i++) {       // every matrix starts a row group of its own
    if (i > 0) { p.seg_end[i - 1] = p.n_row_groups; p.w2[i - 1] = ws[i]->data; p.bias2[i - 1] = ws[i]->bias; p.rows2[i - 1] = (int)ws[i]->rows; p.y_off2[i - 1] = y_off[i] - y_off[0]; }
    p.n_row_groups += (int)((ws[i]->rows + 128 * rt - 1) / (128 * rt));
  }
  if (swiglu_half) p.n_row_groups = (swiglu_half + 127) / 128;   // 128 up rows and their gate rows per work-group
  p.n_tok_tiles = (n_tok + tt * 32 - 1) / (tt * 32);
  const size_t lds = (size_t)tt * 32 * (PF_LDX + 8) * 2 * 2 + (size_t)4 * rt * 2 * 32 * 4;
  static bool attr_done = false;
  if (!attr_done) {
    const void* ks[6] = {(const void*)gemm_q4k_pf<1, 1, CAI_Q4_K>, (const void*)gemm_q4k_pf<2, 1, CAI_Q4_K>, (const void*)gemm_q4k_pf<1, 2, CAI_Q4_K>,
                         (const void*)gemm_q4k_pf<1, 1, CAI_Q5_K>, (const void*)gemm_q4k_pf<2, 1, CAI_Q5_K>, (const void*)gemm_q4k_pf<1, 2, CAI_Q5_K>};
    for (const void* k : ks) if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess) (void)hipGetLastError();
    attr_done = true;
  }
  const int grid = 8 * p.n_tok_tiles * ((p.n_row_groups + 7) / 8);
  if (w->qtype == CAI_Q5_K) {
    if (mode == 3) hipLaunchKernelGGL((gemm_q4k_pf<1, 2, CAI_Q5_K>), dim3(grid), dim3(256), lds, ctx().stream, p);
    else if (mode == 1) hipLaunchKernelGGL((gemm_q4k_pf<1, 1, CAI_Q5_K>), dim3(grid), dim3(256), lds, ctx().stream, p);
    else hipLaunchKernelGGL((gemm_q4k_pf<2, 1, CAI_Q5_K>), dim3(grid), dim3(256), lds, ctx().stream, p);
  } else if (mode == 3) hipLaunchKernelGGL((gemm_q4k_pf<1, 2, CAI_Q4_K>), dim3(grid), dim3(256), lds, ctx().stream, p);
  else if (mode == 1) hipLaunchKernelGGL((gemm_q4k_pf<1, 1, CAI_Q4_K>), dim3(grid), dim3(256), lds, ctx().stream, p);
  else hipLaunchKernelGGL((gemm_q4k_pf<2, 1, CAI_Q4_K>), dim3(grid), dim3(256), lds, ctx().stream, p);
  return CAI_OK;
}

}  // namespace cai

// ------------------------------------------------------------------------------------------
// workspace + C ABI
// ------------------------------------------------------------------------------------------
namespace cai {
struct PrefillWs { _Float16* hi = nullptr; _Float16* lo = nullptr; float* sinv = nullptr; _Float16* sxhi = nullptr; _Float16* sxlo = nullptr; size_t cap_elems = 0; int cap_tok = 0; };
static PrefillWs g_pws;

// Grows the shared activation workspace to n_tok x K (never inside a stream capture).
static int prefill_reserve(int n_tok, int K)
{
  const size_t need = (size_t)n_tok * K;
  if (need > g_pws.cap_elems || n_tok > g_pws.cap_tok) {
    CAI_HIP(hipStreamSynchronize(ctx().stream));
    void* old[] = {g_pws.hi, g_pws.lo, g_pws.sinv, g_pws.sxhi, g_pws.sxlo};
    for (void* q : old) if (q) (void)hipFree(q);
    const size_t ce = std::max(need, g_pws.cap_elems); const int ct = std::max(n_tok, g_pws.cap_tok);
    g_pws = PrefillWs();
    CAI_HIP(hipMalloc((void**)&g_pws.hi, ce * 2)); CAI_HIP(hipMalloc((void**)&g_pws.lo, ce * 2));
    CAI_HIP(hipMalloc((void**)&g_pws.sxhi, ce / 32 * 2 + 64)); CAI_HIP(hipMalloc((void**)&g_pws.sxlo, ce / 32 * 2 + 64));
    CAI_HIP(hipMalloc((void**)&g_pws.sinv, (size_t)ct * 4));
    g_pws.cap_elems = ce; g_pws.cap_tok = ct;
  }
  return CAI_OK;
}

// The planes for n_tok rows of up to K columns in one allocation (a decoder knows its widest row before its first prompt;
// growing width by width would free and allocate, with a stream synchronisation, several times inside that prompt).
int prefill_reserve_rows(int n_tok, int K) { return prefill_reserve(n_tok, K); }

void prefill_release()   // cai_shutdown
{
  void* q[] = {g_pws.hi, g_pws.lo, g_pws.sinv, g_pws.sxhi, g_pws.sxlo};
  for (void* v : q) if (v) (void)hipFree(v);
  g_pws = PrefillWs();
}

int prefill_prep(const float* x, int64_t x_stride, const float* gain, float eps, int K, int n_tok)
{
  int rc;
  if ((rc = prefill_reserve(n_tok, K))) return rc;
  return launch_xprep(x, x_stride, gain, eps, K, n_tok, g_pws.hi, g_pws.lo, g_pws.sinv, g_pws.sxhi, g_pws.sxlo);
}
// planes <- up * silu(gate) of rows holding up | gate (half values each): the pre-pass of the down projection
int prefill_prep_swiglu(const float* gu, int64_t gu_stride, int half, int n_tok)
{
  int rc;
  if ((rc = prefill_reserve(n_tok, half))) return rc;
  xprep_launch<true>(gu, gu_stride, nullptr, 0.0f, half, n_tok, g_pws.hi, g_pws.lo, g_pws.sinv, g_pws.sxhi, g_pws.sxlo);
  return CAI_OK;
}
// Several matrices of one width applied to the prepared activations (q | k | v).
bool prefill_multi_supported(const cai_qw_s* const* ws, int n_w) { return gemm_q4k_multi_supported(ws, n_w) || gemm_blk_multi_supported(ws, n_w); }
int prefill_gemm_multi(const cai_qw_s* const* ws, const int* y_off, int n_w, int n_tok, float* y, int64_t y_stride)
{
  if (n_w > 1 && gemm_q4k_multi_supported(ws, n_w))
    return launch_gemm_q4k_multi(ws, y_off, n_w, g_pws.hi, g_pws.lo, g_pws.sxhi, g_pws.sxlo, g_pws.sinv, n_tok, y, y_stride, nullptr, 0);
  if (n_w > 1 && gemm_blk_multi_supported(ws, n_w))
    return launch_gemm_blk_multi(ws, y_off, n_w, g_pws.hi, g_pws.lo, g_pws.sinv, n_tok, y, y_stride);
  for (int i = 0; i < n_w; i++) {
    const int rc = prefill_gemm(ws[i], n_tok, y + y_off[i], y_stride, nullptr);
    if (rc) return rc;
  }
  return CAI_OK;
}
// y[t][i] = up_i * silu(gate_i) of the prepared activations through a gate|up matrix of 2 * half rows (Q4_K / Q5_K), one launch
bool prefill_gemm_swiglu_supported(const cai_qw_s* w, int n_tok)
{
  // only where the product takes two row tiles per wave anyway (enough work-groups to fill the chip several times over)
  return gemm_mfma_supported(w) && w->qtype != CAI_Q6_K && w->rows % 2 == 0 && (int)((w->rows + 255) / 256) * ((n_tok + 31) / 32) >= 4 * ctx().n_cu;
}
int prefill_gemm_swiglu(const cai_qw_s* w, int n_tok, float* y, int64_t y_stride)
{
  const int zero = 0;
  return launch_gemm_q4k_multi(&w, &zero, 1, g_pws.hi, g_pws.lo, g_pws.sxhi, g_pws.sxlo, g_pws.sinv, n_tok, y, y_stride, nullptr, (int)(w->rows / 2));
}
void prefill_planes(const _Float16** hi, const _Float16** lo, const float** sinv) { *hi = g_pws.hi; *lo = g_pws.lo; *sinv = g_pws.sinv; }
int prefill_gemm(const cai_qw_s* w, int n_tok, float* y, int64_t y_stride, const float* residual)
{
  if (gemm_blk_supported(w)) return launch_gemm_blk(w, g_pws.hi, g_pws.lo, g_pws.sinv, n_tok, y, y_stride, residual);
  return launch_gemm_q4k(w, g_pws.hi, g_pws.lo, g_pws.sxhi, g_pws.sxlo, g_pws.sinv, n_tok, y, y_stride, residual);
}

// Which kernel family takes n_tok tokens of this matrix: 1 = small-batch matrix-core kernel (passes of up to 8 or 16 tokens;
// the bandwidth-bound regime), 2 = prompt kernel on prepared activation planes, 0 = matrix-vector kernel in passes of 8.
//   Q4_K, Q6_K: up to 16 tokens small-batch, above that the prompt kernel;
//   Q8_0, Q4_0: above 16 tokens the prompt kernel; below, small-batch only for a matrix too large for the cache (a small
//               one stays resident: one VALU launch per 8 tokens is cheaper than three launches);
//   per-row int8: small-batch for a large matrix.
int prompt_route(const cai_qw_s* w, int n_tok)
{
  if (gemm_mfma_supported(w)) return n_tok <= 16 && nb_supported(w) ? 1 : 2;
  if (gemm_blk_supported(w) && n_tok > 16) return 2;
  if (nb_supported(w) && w->data_bytes >= ((int64_t)16 << 20)) return 1;
  return 0;
}

// y[t][rows] = W x[t] (+bias) (+residual) for n_tok tokens; x rows are x_stride apart; gain != null fuses RMSNorm.
int prefill_linear(const cai_qw_s* w, const float* x, int64_t x_stride, const float* gain, float eps, int n_tok,
                   float* y, int64_t y_stride, const float* residual)
{
  int rc;
  // few tokens (the bandwidth-bound regime) of a Q4_K or Q6_K matrix, or a large matrix of a type without a prompt kernel (a small
  // one stays in the cache: the single-launch VALU kernel per 8 tokens is cheaper than three launches)
  if (prompt_route(w, n_tok) == 1) return nb_linear(w, x, x_stride, gain, eps, n_tok, y, y_stride, residual);
  if (prompt_route(w, n_tok) == 2) {
    if ((rc = prefill_prep(x, x_stride, gain, eps, (int)w->cols, n_tok))) return rc;
    return prefill_gemm(w, n_tok, y, y_stride, residual);
  }
  // other weight types and small matrices at few tokens: groups of up to 8 tokens through the small-batch kernel (x must be contiguous)
  if (x_stride != w->cols) return set_error(CAI_ERR_UNSUPPORTED, "prefill linear: strided input needs a matrix the matrix-core kernels take");
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
  CAI_ENTER();
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
  if ((flags & CAI_MATRIX_CORES) && nb_supported(w) && !gemm_mfma_supported(w)) rc = nb_linear(w, dx, w->cols, nullptr, 0.0f, n_tokens, dy, w->rows, nullptr);
  else rc = prefill_linear(w, dx, w->cols, nullptr, 0.0f, n_tokens, dy, w->rows, nullptr);
  if (rc) return rc;
  CAI_HIP(hipGetLastError());
  if (!(flags & CAI_Y_DEVICE)) { CAI_HIP(hipMemcpyAsync(y, dy, yb, hipMemcpyDeviceToHost, c.stream)); CAI_HIP(hipStreamSynchronize(c.stream)); }
  return CAI_OK;
}
