// Small-batch (2..8 tokens) Q4_K linear layer on the matrix cores, register-resident form: the decode step of a few sequences
// with ONE launch per linear layer (no activation pre-pass, no slice reduction launch).
//
// The arithmetic is that of gemm_q4k_nb (cai_gemm_nb.hip): A operand = sc_j * q (exact in f16), B operand = the activations
// of up to 8 tokens, scaled per (token, 256-block) by a power of two and split hi + lo into two f16 = the 16 columns of
// v_mfma_f32_16x16x32_f16, one more MFMA per row set and super-block for the - dmin * mn_j * sum_j(x) term
// (Q4_K: neural/neuralgguf.pas:472-514).  What differs is who holds what:
//   * a WAVE owns two super-blocks (512 columns) of EVERY row its work-group walks, so the B operands of its 16 MFMA steps
//     never change: it reads its 8 x 512 activations as fp32 once, applies the RMSNorm gain, finds the block scales, splits
//     hi + lo and keeps the operands in 64 registers for the whole launch - no activation planes in memory, no LDS traffic
//     in the product loop, no barrier before the first product;
//   * a work-group = the waves that together cover the columns (7 waves for 3584) walks 32-row pairs of row sets; per pair
//     every wave leaves its share in LDS, one barrier, and ONE wave (taking turns) adds the shares in wave order and
//     finishes the rows: 1/rms of the token (sums of squares exchanged through LDS), bias, residual, or SwiGLU when the two
//     row sets of a pair are 16 up rows and their 16 gate rows - written once, as fp32, where the next launch reads them;
//   * a width of more than 16 super-blocks (the 18944-wide down projection) is cut into column slices = work-groups of
//     blockIdx.y; the slices' shares meet in a partial buffer and the LAST slice work-group of a row group to arrive (an
//     arrival counter, as in the attention merge) adds them in slice order with bias and residual.
// Fixed orders everywhere: the result does not depend on timing.
#include "cai_internal.hpp"
#include "cai_gemv_common.hpp"
#include <algorithm>

namespace cai {

namespace {
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int RA_TK = 8;         // tokens per launch
constexpr int RA_NW = 8;         // waves per work-group at most
constexpr int RA_SBW = 2;        // super-blocks of a row per wave
constexpr int RA_SMAX = RA_NW * RA_SBW;   // super-blocks per column slice at most
constexpr int RA_BB = 144;       // bytes of a Q4_K super-block
constexpr int RA_PART_BATCH = 8; // slices of an element the last arriver requests at once (times 2 elements, times 2 for SwiGLU)
constexpr int RA_XLD = RA_SBW * 256 + 8;          // halfs per operand column in LDS (+8: 16 columns x 16-byte reads tile the banks)
constexpr int RA_WAVE_LDS = 16 * RA_XLD * 2 + 16 * 16 * 2 + RA_SBW * RA_TK * 4 + 192;   // = 17408 bytes per wave

struct RaSeg { const uint8_t* w; const float* bias; int rows; int y_off; int pair_end; };   // pair_end: cumulative 32-row pairs

struct RaParams {
  RaSeg seg[3]; int n_seg;                       // up to three matrices of equal width share a launch (q | k | v)
  float eps;                                     // RMSNorm of the activations (when a gain is given): 1/rms is applied to the result
  int swiglu_half;                               // > 0: rows [0, half) are up, [half, 2 half) gate; pair p = up rows 16 p.. + gate rows half + 16 p..
  float* y; long long y_stride; const float* residual;   // residual: laid out like y (may be y itself)
  int n_slices;
  float* part; long long part_stride;            // n_slices > 1: part[(slice * n_tok + t) * part_stride + y_off + row]
  unsigned* counters;                            // n_slices > 1: one arrival counter per row group (blockIdx.x), wrapping to 0
  unsigned long long* timeline;                  // stamps of this launch's work-groups (null: none)
};

__device__ __forceinline__ void ra_part_store(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float ra_part_load(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// The weight operand of one MFMA step from two quant dwords (8 bytes, low or high nibbles): with K = 0x64006400 the halfs of
// (d & 0x000f000f) | K are 1024 + the low nibbles of bytes 0 and 2, those of (d & 0x00f000f0) | K are 1024 + 16 x the high
// nibbles of the same bytes (no shift needed); d >> 8 gives bytes 1 and 3.  One packed fma each turns them into the exact
// halfs sc * q: (1024 + q) * sc - 1024 * sc, or (1024 + 16 q) * (sc / 16) - 64 * sc.  The order in which the 8 weights land in
// the operand (bytes 0, 2, 1, 3 of the first dword, then of the second) is the order the activation operand is built in.
// (written as a bit-field insert into a register copy of K - (d & M) | (K & ~M) - so that it is ONE instruction, v_bfi_b32:
// with two literal constants the and and the or stay separate.)
template <bool HIGH> __device__ __forceinline__ half8_t ra_weights(uint32_t d0, uint32_t d1, half2_t s2, half2_t c2, uint32_t kreg)
{
  constexpr uint32_t M = HIGH ? 0x00f000f0u : 0x000f000fu;
  const uint32_t e0 = d0 >> 8, e1 = d1 >> 8;
  const half2_t a0 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, (d0 & M) | (kreg & ~M)), s2, c2);
  const half2_t a1 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, (e0 & M) | (kreg & ~M)), s2, c2);
  const half2_t a2 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, (d1 & M) | (kreg & ~M)), s2, c2);
  const half2_t a3 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, (e1 & M) | (kreg & ~M)), s2, c2);
  return half8_t{a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
}
// all-reduce over the 16 lanes of a row: lane ^ 1, lane ^ 2, then the mirror images within 8 and within 16
#define RA_DPP(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xf, 0xf, false))
__device__ __forceinline__ float ra_row_max(float v)
{
  v = fmaxf(v, RA_DPP(v, 0xb1)); v = fmaxf(v, RA_DPP(v, 0x4e)); v = fmaxf(v, RA_DPP(v, 0x141)); v = fmaxf(v, RA_DPP(v, 0x140));
  return v;
}
__device__ __forceinline__ float ra_row_sum(float v)
{
  v += RA_DPP(v, 0xb1); v += RA_DPP(v, 0x4e); v += RA_DPP(v, 0x141); v += RA_DPP(v, 0x140);
  return v;
}
// all-reduce over each half of a row (8 lanes)
__device__ __forceinline__ float ra_oct_sum(float v)
{
  v += RA_DPP(v, 0xb1); v += RA_DPP(v, 0x4e); v += RA_DPP(v, 0x141);
  return v;
}
// the value of lane ^ 8 (the other half of a 16-lane row: the hi / lo column of the same token)
__device__ __forceinline__ float ra_ror8(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false)); }
__device__ __forceinline__ uint32_t ra_ror8(uint32_t v) { return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x128, 0xf, 0xf, false); }
}  // namespace

// v_mfma_f32_16x16x32_f16: lane (m = lane % 16, kg = lane / 16) supplies 8 consecutive k of row m (A) / column m (B); the
// 16 x 16 result has rows 4 kg .. 4 kg + 3 of column m in this lane.  The order of k inside a super-block is free (both
// operands follow it) and is chosen for the weight requests: the four kg lanes of a row ask for 64 contiguous quant bytes per
// request (bytes 16 kg .. + 15, then 64 + 16 kg .. + 15).  With g = kg / 2 and c1 = kg % 2 lane kg owns weights
// 16 c1 .. 16 c1 + 15 of sub-blocks 2 g + 4 c + nib (c = request, nib = low / high nibbles), step t = 4 c + 2 nib + j takes
// the 8 of them at 8 j (in the order 0, 2, 1, 3, 4, 6, 5, 7: see ra_weights).  For the min term lane kg stands for the two sub-blocks 2 g + 4 c1, + 1 (each lane pair kg, kg ^ 1
// holds the halves of four sub-blocks' activations, so their sums are one exchange away).
// (what the first requests need travels as leading scalar arguments, preloaded in scalar registers)
// HH: 16-row sets per unit of rows (2: pairs - what SwiGLU needs and what long walks take; 1 halves the unit, for products
// with fewer pairs than compute units or an uneven number per work-group).  GAIN: the activations carry an RMSNorm gain.
template <int HH, bool GAIN>
__global__ __launch_bounds__(64 * RA_NW) void gemm_q4k_ra(const float* hsrc, const long long hstride, const float* hgain, const int hcols, const int hntok,
                                                          const int hnpairs, const int hS, const RaParams p)
{
  // per wave RA_WAVE_LDS bytes: the operand columns [16][RA_XLD] halfs while the activations are converted (each wave converts
  // and reads back only its own columns: no work-group barrier), their sub-block sums [16][16] halfs and 1 / scale [2][8]; once
  // the operands are in registers the first 2 KB are the wave's shares of the pair in hand: [2 parities][32 lanes][8]
  extern __shared__ __align__(16) unsigned char ra_dyn[];
  __shared__ __align__(16) float s_d[RA_NW][2][32];         // d, 32 * dmin per row of the item in hand
  __shared__ float ssq_s[RA_SMAX][RA_TK];
  __shared__ int s_is_last;
  const unsigned long long tl0 = timeline_now();
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, kg = lane >> 4, g = kg >> 1, c1 = kg & 1;
  const int K = hcols, nsb = K >> 8;
  const int slice = blockIdx.y, sb0 = slice * hS, nS = min(hS, nsb - sb0);
  const int nwa = (nS + RA_SBW - 1) / RA_SBW;                              // waves of this work-group with columns to cover
  const int nsw = max(0, min(RA_SBW, nS - RA_SBW * wave));                  // super-blocks of this wave
  const int sbw0 = sb0 + min(RA_SBW * wave, nS - 1);                        // its first one (an idle wave re-reads the last)
  const int64_t row_bytes = (int64_t)nsb * RA_BB;
  const int npw = (int)blockIdx.x < hnpairs ? (hnpairs - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;   // pairs of this work-group
  const int nq = RA_SBW * npw;                                              // (pair, super-block) items of a wave
  const int tok = n & (RA_TK - 1), tokc = min(tok, hntok - 1);
  const bool tok_on = tok < hntok;
  const bool lo_col = n >= RA_TK;

  // rows of a pair: plain matrices take 32 consecutive rows of a segment, SwiGLU 16 up rows and their 16 gate rows
  auto locate = [&](int pair, const RaSeg*& sg, int& r0, int& r1) __attribute__((always_inline)) {
    int sgi = 0, t0 = 0;
    if (p.n_seg > 1 && pair >= p.seg[0].pair_end) { sgi = 1; t0 = p.seg[0].pair_end; }
    if (p.n_seg > 2 && pair >= p.seg[1].pair_end) { sgi = 2; t0 = p.seg[1].pair_end; }
    sg = &p.seg[sgi];
    if (p.swiglu_half > 0) { r0 = 16 * pair; r1 = p.swiglu_half + 16 * pair; }
    else { r0 = (pair - t0) * 16 * HH; r1 = r0 + 16; }
  };

  struct WRegs { uint4 h[HH], q[HH][2]; };
  // weights of item q = (pair q / 2, super-block q % 2 of this wave): for the rows n of both row sets the header and this
  // lane's 2 x 16 quant bytes.  Loads are never conditional: past the last item the last one is fetched again (a cache hit).
  auto load_w = [&](int q, WRegs& r) __attribute__((always_inline)) {
    const int qc = max(min(q, nq - 1), 0);
    const int pair = min((int)blockIdx.x + (qc >> 1) * (int)gridDim.x, hnpairs - 1), sb = sbw0 + min(qc & 1, max(nsw, 1) - 1);
    const RaSeg* sg; int r0, r1; locate(pair, sg, r0, r1);
#pragma unroll
    for (int hh = 0; hh < HH; hh++) {
      const uint8_t* blk = sg->w + (int64_t)min((hh ? r1 : r0) + n, sg->rows - 1) * row_bytes + (int64_t)sb * RA_BB;   // tail rows: re-read the last row
      r.h[hh] = *reinterpret_cast<const uint4*>(blk);
      r.q[hh][0] = *reinterpret_cast<const uint4*>(blk + 16 + 16 * kg);
      r.q[hh][1] = *reinterpret_cast<const uint4*>(blk + 80 + 16 * kg);
    }
  };
  WRegs wa, wb, wc, wd;

  // ---- this wave's activations: 8 tokens x its super-blocks, requested before the first weights ----
  // Requests in memory order: lane (r = lane / 16, i = lane % 16) asks for floats 64 m + 4 i .. + 3 (m = 0..3) of super-block j
  // of tokens r and 4 + r, so a request covers 256 contiguous bytes of each of four tokens (in operand order a request would
  // touch 64 different cache lines).  A 16-lane row then holds whole (token, block)s: scale and sums are row-local reductions.
  unsigned char* wl = ra_dyn + (size_t)wave * RA_WAVE_LDS;
  _Float16* xw = reinterpret_cast<_Float16*>(wl);                          // [16 columns][RA_XLD]
  _Float16* sxw = xw + 16 * RA_XLD;                                        // [16 columns][16 sub-blocks]
  float* sinvw = reinterpret_cast<float*>(sxw + 16 * 16);                  // [RA_SBW][8 tokens]
  const int rr = lane >> 4, ii = lane & 15;
  float4 xr[RA_SBW][2][4];
#pragma unroll
  for (int j = 0; j < RA_SBW; j++)
#pragma unroll
    for (int hq = 0; hq < 2; hq++) {
      const float* px = hsrc + (int64_t)min(4 * hq + rr, hntok - 1) * hstride + (int64_t)(sbw0 + min(j, max(nsw, 1) - 1)) * 256 + 4 * ii;
#pragma unroll
      for (int m = 0; m < 4; m++) xr[j][hq][m] = *reinterpret_cast<const float4*>(px + 64 * m);
    }
  float4 gr[RA_SBW][4];
#pragma unroll
  for (int j = 0; j < RA_SBW; j++) {
    const float* pg = (GAIN ? hgain : hsrc) + (int64_t)(sbw0 + min(j, max(nsw, 1) - 1)) * 256 + 4 * ii;    // (no gain: any readable address, the values are not used)
#pragma unroll
    for (int m = 0; m < 4; m++) gr[j][m] = *reinterpret_cast<const float4*>(pg + 64 * m);
  }
  load_w(0, wa); load_w(1, wb);
  timeline_put(p.timeline, 0, tl0); timeline_stamp(p.timeline, 1);

#pragma unroll
  for (int j = 0; j < RA_SBW; j++)
#pragma unroll
    for (int hq = 0; hq < 2; hq++) {
      const int t8 = 4 * hq + rr;                 // the row's token
      float v[4][4];
      float amax = 0.0f, ss = 0.0f;
#pragma unroll
      for (int m = 0; m < 4; m++) {
        const float4 a = xr[j][hq][m], gq = gr[j][m];
        const float raw[4] = {a.x, a.y, a.z, a.w}, gg[4] = {gq.x, gq.y, gq.z, gq.w};
#pragma unroll
        for (int u = 0; u < 4; u++) { v[m][u] = GAIN ? raw[u] * gg[u] : raw[u]; amax = fmaxf(amax, fabsf(v[m][u])); ss = fmaf(raw[u], raw[u], ss); }
      }
      amax = ra_row_max(amax); ss = ra_row_sum(ss);
      if (j == 0 && hq == 0) timeline_stamp_after(p.timeline, 2, amax);
      int e = 0;
      if (amax > 0.0f && amax < 3.0e38f) { int ex; frexpf(amax, &ex); e = 14 - ex; }   // amax * 2^e in [2^13, 2^14)
      e = max(-60, min(60, e));
      const bool on = t8 < hntok;
      const float s = on ? ldexpf(1.0f, e) : 0.0f;      // (an absent token's columns: zeros)
#pragma unroll
      for (int m = 0; m < 4; m++) {
        // vs = h + l to 21 bits, both parts converted two at a time towards zero (v_cvt_pkrtz_f16_f32: the pair comes out packed, and
        // in the operand's order - inside a group of 8 that order is 0, 2, 1, 3, 4, 6, 5, 7 (ra_weights): the middle two of every four
        // swap); l = vs - h is exact in fp32 and has the sign of vs
        float vs[4], sm = 0.0f;
#pragma unroll
        for (int u = 0; u < 4; u++) { vs[u] = v[m][u] * s; sm += vs[u]; }
        typedef __fp16 pk2_t __attribute__((ext_vector_type(2)));
        const pk2_t h02 = __builtin_amdgcn_cvt_pkrtz(vs[0], vs[2]), h13 = __builtin_amdgcn_cvt_pkrtz(vs[1], vs[3]);
        const pk2_t l02 = __builtin_amdgcn_cvt_pkrtz(vs[0] - (float)h02.x, vs[2] - (float)h02.y), l13 = __builtin_amdgcn_cvt_pkrtz(vs[1] - (float)h13.x, vs[3] - (float)h13.y);
        *reinterpret_cast<uint2*>(xw + t8 * RA_XLD + j * 256 + 64 * m + 4 * ii) = make_uint2(__builtin_bit_cast(uint32_t, h02), __builtin_bit_cast(uint32_t, h13));
        *reinterpret_cast<uint2*>(xw + (8 + t8) * RA_XLD + j * 256 + 64 * m + 4 * ii) = make_uint2(__builtin_bit_cast(uint32_t, l02), __builtin_bit_cast(uint32_t, l13));
        // sub-block 2 m + i / 8 of the block: the sum of 8 lanes' values, / 32, hi + lo
        sm = ra_oct_sum(sm) * 0.03125f;
        const _Float16 qh = (_Float16)sm, ql = (_Float16)(sm - (float)qh);
        if ((ii & 7) == 0) { sxw[t8 * 16 + j * 8 + 2 * m + (ii >> 3)] = qh; sxw[(8 + t8) * 16 + j * 8 + 2 * m + (ii >> 3)] = ql; }
      }
      if (ii == 0) {
        sinvw[j * RA_TK + t8] = on ? ldexpf(1.0f, -e) : 0.0f;
        if (j < nsw) ssq_s[RA_SBW * wave + j][t8] = ss;
      }
    }
  __builtin_amdgcn_wave_barrier();    // LDS operations of a wave complete in order: its own columns are there
  // the operands in MFMA order: column n, this lane's 8 k of every step
  half8_t Bx[RA_SBW][8]; half2_t bm[RA_SBW]; float sinv[RA_SBW];
#pragma unroll
  for (int j = 0; j < RA_SBW; j++) {
#pragma unroll
    for (int t = 0; t < 8; t++)
      Bx[j][t] = *reinterpret_cast<const half8_t*>(xw + n * RA_XLD + j * 256 + 64 * g + 16 * c1 + 128 * (t >> 2) + 32 * ((t >> 1) & 1) + 8 * (t & 1));
    bm[j] = *reinterpret_cast<const half2_t*>(sxw + n * 16 + j * 8 + 2 * g + 4 * c1);    // sub-blocks 2 g + 4 c1, + 1
    sinv[j] = sinvw[j * RA_TK + tok];
  }
  __builtin_amdgcn_wave_barrier();    // (the region is written again as the wave's shares of a pair)
  load_w(2, wc);
  timeline_stamp_after(p.timeline, 3, sinv[RA_SBW - 1]);
  timeline_stamp(p.timeline, 4);
  // what the finishing wave of a pair adds to the rows (bias, residual) is requested when the pair starts: by every wave, so
  // that the requests stay unconditional (a kilobyte per wave and pair), and from a harmless address when there is none
  struct Extra { float4 bias[HH], res[HH]; };
  auto prefetch = [&](int i, Extra& f) __attribute__((always_inline)) {
    const int pair = min((int)blockIdx.x + min(i, max(npw, 1) - 1) * (int)gridDim.x, hnpairs - 1);
    const RaSeg* sg; int r0, r1; locate(pair, sg, r0, r1);
#pragma unroll
    for (int hh = 0; hh < HH; hh++) {
      const int row = (hh ? r1 : r0) + 4 * kg;
      const float* bp = sg->bias ? sg->bias + row : reinterpret_cast<const float*>(sg->w);
      const float* rp = p.residual ? p.residual + (int64_t)tokc * p.y_stride + sg->y_off + row : p.y;
      f.bias[hh] = *reinterpret_cast<const float4*>(bp);
      f.res[hh] = *reinterpret_cast<const float4*>(rp);
    }
  };
  Extra ea, eb;
  float acc[HH][4];
  const _Float16 k1024 = (_Float16)1024.0f, kz = (_Float16)0.0f;
  uint32_t kreg = 0x64006400u;                 // 1024.0 twice, kept in a register the compiler cannot fold (see ra_weights)
  asm volatile("" : "+v"(kreg));

  auto compute = [&](const WRegs& r, const int j) __attribute__((always_inline)) {
    if (j == 0) {
#pragma unroll
      for (int hh = 0; hh < HH; hh++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[hh][i] = 0.0f;
    }
    if (j >= nsw) return;
    float4_t C[HH], Cm[HH];
    half2_t s2[HH][4], c2[HH][4];
#pragma unroll
    for (int hh = 0; hh < HH; hh++) {
      // 6-bit scales / mins (neural/neuralgguf.pas:448-464), one per byte: sub-blocks 0..3 and 4..7
      const uint4 h = r.h[hh];
      const uint32_t sc_lo = h.y & 0x3f3f3f3fu, sc_hi = (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u);
      const uint32_t mn_lo = h.z & 0x3f3f3f3fu, mn_hi = ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u);
      const uint32_t scq[2] = {sc_lo >> (16 * g), sc_hi >> (16 * g)};       // bytes 0, 1 = sub-blocks 2 g + 4 c, + 1
      const uint32_t mnp = (c1 ? mn_hi : mn_lo) >> (16 * g);                // sub-blocks 2 g + 4 c1, + 1
      const half2_t mnh = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, mnp, 0x04010400u)) - half2_t{k1024, k1024};
#pragma unroll
      for (int c = 0; c < 2; c++) {
        // low nibbles: (sc, -1024 sc); high nibbles arrive as 16 q: (sc / 16, -64 sc) - all exact in f16
        const half2_t sch = (__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, scq[c], 0x04010400u)) - half2_t{k1024, k1024}) * half2_t{(_Float16)1.0f, (_Float16)0.0625f};
        const half2_t cch = sch * half2_t{(_Float16)(-1024.0f), (_Float16)(-1024.0f)};
        s2[hh][2 * c] = half2_t{sch.x, sch.x}; s2[hh][2 * c + 1] = half2_t{sch.y, sch.y};
        c2[hh][2 * c] = half2_t{cch.x, cch.x}; c2[hh][2 * c + 1] = half2_t{cch.y, cch.y};
      }
      if (kg == 0) {
        const float d = __half2float(__ushort_as_half((unsigned short)(h.x & 0xffffu)));
        const float dmin = __half2float(__ushort_as_half((unsigned short)(h.x >> 16)));
        s_d[wave][0][16 * hh + n] = d; s_d[wave][1][16 * hh + n] = dmin * 32.0f;
      }
      // - dmin * mn * (sum of the sub-block's activations): k = this lane's two sub-blocks, the other six k stay zero
      const half8_t Am = {mnh.x, mnh.y, kz, kz, kz, kz, kz, kz}, Bm = {bm[j].x, bm[j].y, kz, kz, kz, kz, kz, kz};
      const float4_t z4 = {0.0f, 0.0f, 0.0f, 0.0f};
      Cm[hh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Am, Bm, z4, 0, 0, 0);
      C[hh] = z4;
    }
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const int c = t >> 2, nib = (t >> 1) & 1, jj = t & 1;      // request, nibble, dword pair
#pragma unroll
      for (int hh = 0; hh < HH; hh++) {
        const uint4& qq = r.q[hh][c];
        const uint32_t d0 = jj ? qq.z : qq.x, d1 = jj ? qq.w : qq.y;
        const half8_t A = nib ? ra_weights<true>(d0, d1, s2[hh][2 * c + 1], c2[hh][2 * c + 1], kreg) : ra_weights<false>(d0, d1, s2[hh][2 * c], c2[hh][2 * c], kreg);
        C[hh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Bx[j][t], C[hh], 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();   // s_d was written by this wave's own lanes above; LDS operations of a wave complete in order
#pragma unroll
    for (int hh = 0; hh < HH; hh++) {
      const float4 d4 = *reinterpret_cast<const float4*>(&s_d[wave][0][16 * hh + 4 * kg]);
      const float4 m4 = *reinterpret_cast<const float4*>(&s_d[wave][1][16 * hh + 4 * kg]);
      acc[hh][0] += sinv[j] * (d4.x * C[hh][0] - m4.x * Cm[hh][0]);
      acc[hh][1] += sinv[j] * (d4.y * C[hh][1] - m4.y * Cm[hh][1]);
      acc[hh][2] += sinv[j] * (d4.z * C[hh][2] - m4.z * Cm[hh][2]);
      acc[hh][3] += sinv[j] * (d4.w * C[hh][3] - m4.w * Cm[hh][3]);
    }
    __builtin_amdgcn_wave_barrier();
  };

  // ---- end of a pair: every wave leaves its share (column t hi + column 8 + t lo), one wave finishes the rows ----
  auto pair_end = [&](int i, const Extra& f) __attribute__((always_inline)) {
    const int slot = i & 1;
    if (nsw > 0) {
      float tot[4 * HH];
#pragma unroll
      for (int hh = 0; hh < HH; hh++)
#pragma unroll
        for (int k = 0; k < 4; k++) tot[4 * hh + k] = acc[hh][k] + ra_ror8(acc[hh][k]);
      if (!lo_col) {
        float* dst = reinterpret_cast<float*>(wl) + (slot * 32 + kg * 8 + n) * 8;
        *reinterpret_cast<float4*>(dst) = make_float4(tot[0], tot[1], tot[2], tot[3]);
        if constexpr (HH == 2) *reinterpret_cast<float4*>(dst + 4) = make_float4(tot[4], tot[5], tot[6], tot[7]);
      }
    }
    __syncthreads();     // (the slot is written again two pairs on: after the next barrier, which the finishing wave reaches after its reads)
    if (wave != i % nwa || lo_col) return;
    float t8[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int w = 0; w < nwa; w++) {       // wave order: fixed
      const float* src = reinterpret_cast<const float*>(ra_dyn + (size_t)w * RA_WAVE_LDS) + (slot * 32 + kg * 8 + n) * 8;
      const float4 a = *reinterpret_cast<const float4*>(src);
      t8[0] += a.x; t8[1] += a.y; t8[2] += a.z; t8[3] += a.w;
      if constexpr (HH == 2) { const float4 b = *reinterpret_cast<const float4*>(src + 4); t8[4] += b.x; t8[5] += b.y; t8[6] += b.z; t8[7] += b.w; }
    }
    if (!tok_on) return;
    const int pair = (int)blockIdx.x + i * (int)gridDim.x;
    const RaSeg* sg; int r0, r1; locate(pair, sg, r0, r1);
    if (p.n_slices > 1) {     // a slice's share of the rows (finished by the last slice to arrive, below)
#pragma unroll
      for (int hh = 0; hh < HH; hh++) {
        float* dst = p.part + ((int64_t)slice * hntok + tok) * p.part_stride + sg->y_off + (hh ? r1 : r0) + 4 * kg;
#pragma unroll
        for (int k = 0; k < 4; k++) ra_part_store(dst + k, t8[4 * hh + k]);
      }
      return;
    }
    float inv = 1.0f;
    if (GAIN) {   // (a product with a gain is one slice: the work-group has seen the whole row; every wave has passed this pair's barrier)
      float t = 0.0f;
      for (int sb = 0; sb < nS; sb++) t += ssq_s[sb][tok];     // fixed order
      inv = 1.0f / sqrtf(t / (float)K + p.eps);
    }
    if (HH == 2 && p.swiglu_half > 0) {
      const int col = 16 * pair + 4 * kg;       // rows r0 + 4 kg .. + 3 (up) and r1 + 4 kg .. + 3 (gate)
      const float bu[4] = {f.bias[0].x, f.bias[0].y, f.bias[0].z, f.bias[0].w}, bg[4] = {f.bias[HH - 1].x, f.bias[HH - 1].y, f.bias[HH - 1].z, f.bias[HH - 1].w};
      float o[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        float up = inv * t8[k], gate = inv * t8[4 + k];
        if (sg->bias) { up += bu[k]; gate += bg[k]; }
        o[k] = silu_mul(up, gate);
      }
      *reinterpret_cast<float4*>(p.y + (int64_t)tok * p.y_stride + col) = make_float4(o[0], o[1], o[2], o[3]);
      return;
    }
#pragma unroll
    for (int hh = 0; hh < HH; hh++) {
      const int row = (hh ? r1 : r0) + 4 * kg;
      const float bb[4] = {f.bias[hh].x, f.bias[hh].y, f.bias[hh].z, f.bias[hh].w}, rr[4] = {f.res[hh].x, f.res[hh].y, f.res[hh].z, f.res[hh].w};
      float vv[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        vv[k] = inv * t8[4 * hh + k];
        if (sg->bias) vv[k] += bb[k];
        if (p.residual) vv[k] += rr[k];
      }
      *reinterpret_cast<float4*>(p.y + (int64_t)tok * p.y_stride + sg->y_off + row) = make_float4(vv[0], vv[1], vv[2], vv[3]);
    }
  };

  for (int q = 0; q < nq; q += 4) {
    prefetch(q >> 1, ea);
    load_w(q + 3, wd); compute(wa, 0);
    load_w(q + 4, wa); compute(wb, 1);
    if (q == 0 && p.n_slices == 1) timeline_stamp_after(p.timeline, 6, acc[0][0]);
    pair_end(q >> 1, ea);
    prefetch((q >> 1) + 1, eb);
    load_w(q + 5, wb); if (q + 2 < nq) compute(wc, 0);      // (requests stay unconditional)
    load_w(q + 6, wc); if (q + 2 < nq) { compute(wd, 1); pair_end((q >> 1) + 1, eb); }
  }
  timeline_stamp(p.timeline, 5);
  if (p.n_slices > 1) {
    // the slices of a row group meet: shares stored with agent-scope stores and acknowledged (vmcnt(0)) before the barrier and
    // the work-group's arrival; the last arriver reads them with agent-scope loads, in slice order
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (threadIdx.x == 0)
      s_is_last = __builtin_amdgcn_atomic_inc32(p.counters + blockIdx.x, (unsigned)p.n_slices - 1, __ATOMIC_RELAXED, "agent") == (unsigned)p.n_slices - 1;
    __syncthreads();
    timeline_stamp(p.timeline, 6);
    if (!s_is_last) { timeline_stamp(p.timeline, 7); return; }
    // the elements EB at a time: all slices' shares of a batch of elements (and their bias and residual) are requested before
    // the first addition; the additions run in slice order
    const int rpu = 16 * HH;                                  // rows per unit
    const int total = npw * rpu * hntok;
    const int64_t sstep = (int64_t)hntok * p.part_stride;     // from one slice's share of an element to the next
    constexpr int EB = 2;
    for (int e0 = threadIdx.x; e0 < total; e0 += EB * blockDim.x) {
      const float* src[EB]; float bias[EB], res[EB], sum[EB]; int64_t out[EB]; bool on[EB];
#pragma unroll
      for (int b = 0; b < EB; b++) {
        const int e = min(e0 + b * (int)blockDim.x, total - 1);
        on[b] = e0 + b * (int)blockDim.x < total;
        const int rl = e % rpu, t = (e / rpu) % hntok, i = (e / rpu) / hntok;
        const RaSeg* sg; int r0, r1; locate((int)blockIdx.x + i * (int)gridDim.x, sg, r0, r1);
        src[b] = p.part + (int64_t)t * p.part_stride + sg->y_off + r0 + rl;
        out[b] = (int64_t)t * p.y_stride + sg->y_off + r0 + rl;
        bias[b] = sg->bias ? sg->bias[r0 + rl] : 0.0f;
        res[b] = p.residual ? p.residual[out[b]] : 0.0f;
        sum[b] = 0.0f;
      }
      for (int s0 = 0; s0 < p.n_slices; s0 += RA_PART_BATCH) {
        float ps[EB][RA_PART_BATCH];
#pragma unroll
        for (int b = 0; b < EB; b++)
#pragma unroll
          for (int u = 0; u < RA_PART_BATCH; u++) ps[b][u] = ra_part_load(src[b] + (int64_t)min(s0 + u, p.n_slices - 1) * sstep);
#pragma unroll
        for (int b = 0; b < EB; b++)
#pragma unroll
          for (int u = 0; u < RA_PART_BATCH; u++) if (s0 + u < p.n_slices) sum[b] += ps[b][u];
      }
#pragma unroll
      for (int b = 0; b < EB; b++) if (on[b]) p.y[out[b]] = sum[b] + bias[b] + res[b];
    }
  }
  timeline_stamp(p.timeline, 7);
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
namespace {
struct RaWs { float* part = nullptr; size_t cap_part = 0; unsigned* counters = nullptr; int generation = 0; };
RaWs g_ra;
constexpr int RA_COUNTERS = 1024;

// How a product over nsb super-blocks and `pairs` row pairs is cut: column slices of S super-blocks (work-groups of
// ceil(S / 2) waves; a CU holds 8 such waves) and gx row groups, so that all work-groups are resident at once and the
// longest walk (pairs of a work-group) is shortest; fewer slices at equal length.
bool ra_geometry(int nsb, int pairs, int& S, int& n_slices, int& gx)
{
  const int n_cu = ctx().n_cu;
  const int ns_min = (nsb + RA_SMAX - 1) / RA_SMAX;
  float best = 3.0e38f;
  // (a width that fits one slice stays one: no partial results at all)
  for (int ns = ns_min; ns <= (ns_min == 1 ? 1 : std::min(nsb, ns_min + 8)); ns++) {
    const int s = (nsb + ns - 1) / ns;
    if ((nsb + s - 1) / s != ns) continue;
    const int nw = (s + RA_SBW - 1) / RA_SBW;
    const int slots = n_cu * (RA_NW / nw);
    const int g = std::max(1, std::min(pairs, std::min(slots / ns, RA_COUNTERS)));
    // every wave takes two super-blocks of each pair of its work-group: the walk is as long as the pairs per work-group
    const float cost = (float)((pairs + g - 1) / g) + 0.05f * (float)ns;
    if (cost < best) { best = cost; S = s; n_slices = ns; gx = g; }
  }
  return best < 3.0e38f;
}
}  // namespace

void ra_release()
{
  if (g_ra.part) (void)hipFree(g_ra.part);
  if (g_ra.counters) (void)hipFree(g_ra.counters);
  const int gen = g_ra.generation + 1;
  g_ra = RaWs(); g_ra.generation = gen;
}
int ra_ws_generation() { return g_ra.generation; }

// Partial buffer (floats) and arrival counters of the sliced products (never inside a stream capture).
int ra_reserve(size_t part_floats)
{
  if (!g_ra.counters) {
    CAI_HIP(hipMalloc((void**)&g_ra.counters, RA_COUNTERS * sizeof(unsigned)));
    CAI_HIP(hipMemsetAsync(g_ra.counters, 0, RA_COUNTERS * sizeof(unsigned), ctx().stream));
    CAI_HIP(hipStreamSynchronize(ctx().stream));
    g_ra.generation++;
  }
  if (part_floats > g_ra.cap_part) {
    CAI_HIP(hipStreamSynchronize(ctx().stream));
    if (g_ra.part) (void)hipFree(g_ra.part);
    g_ra.part = nullptr; g_ra.cap_part = 0;
    CAI_HIP(hipMalloc((void**)&g_ra.part, part_floats * sizeof(float)));
    g_ra.cap_part = part_floats; g_ra.generation++;
  }
  return CAI_OK;
}

// Floats of partial buffer a product of `rows` outputs over `cols` columns may need for 8 tokens (0: it is one slice)
size_t ra_part_floats(int64_t rows, int64_t cols)
{
  const int nsb = (int)(cols >> 8);
  if (nsb <= RA_SMAX) return 0;
  const int ns_max = (nsb + RA_SMAX - 1) / RA_SMAX + 8;
  return (size_t)ns_max * RA_TK * (size_t)((rows + 3) / 4 * 4);
}

// Whether ra_gemm takes these matrices: Q4_K, one width of whole super-blocks, whole 16-row sets,
// one column slice when the product carries an RMSNorm or SwiGLU.
bool ra_supported(const cai_qw_s* const* ws, int n_w, bool normed, int swiglu_half)
{
  if (n_w < 1 || n_w > 3 || (swiglu_half > 0 && n_w != 1)) return false;
  for (int i = 0; i < n_w; i++) {
    const cai_qw_s* w = ws[i];
    if (w->qtype != CAI_Q4_K || w->cols != ws[0]->cols || w->cols % 256 || w->cols < 256 || w->rows % 16) return false;
  }
  if (swiglu_half > 0 && (ws[0]->rows != 2 * (int64_t)swiglu_half || swiglu_half % 16)) return false;
  // a product with an RMSNorm or SwiGLU must be one column slice (its finishing wave needs the whole row's sum of squares and
  // both halves' rows); measured on 5120 columns a sliced form with those exchanged through memory lost to the plane form
  const int nsb = (int)(ws[0]->cols >> 8);
  return !((normed || swiglu_half > 0) && nsb > RA_SMAX);
}

// y[t][y_off_i + r] = W_i (gain . x_t) / rms(x_t) + bias_i [+ residual]   for t < n_tok <= 8, or, with swiglu_half > 0,
// y[t][r] = up_r * silu(gate_r) of the one matrix [up; gate].  x: fp32 rows of x_stride floats (16-byte aligned).
int ra_gemm(const cai_qw_s* const* ws, const int* y_off, int n_w, int n_tok, const float* x, int64_t x_stride, const float* gain, float eps,
            int swiglu_half, float* y, int64_t y_stride, const float* residual)
{
  if (n_tok < 1 || n_tok > RA_TK || !ra_supported(ws, n_w, gain != nullptr, swiglu_half))
    return set_error(CAI_ERR_UNSUPPORTED, "small-batch product (register form): %d matrices, %d tokens", n_w, n_tok);
  if ((x_stride & 3) || (reinterpret_cast<uintptr_t>(x) & 15) || (gain && (reinterpret_cast<uintptr_t>(gain) & 15)))
    return set_error(CAI_ERR_INVALID, "small-batch product (register form): activations must be 16-byte aligned rows");
  if ((y_stride & 3) || (reinterpret_cast<uintptr_t>(y) & 15) || (residual && (reinterpret_cast<uintptr_t>(residual) & 15)))
    return set_error(CAI_ERR_INVALID, "small-batch product (register form): results must be 16-byte aligned rows");
  for (int i = 0; i < n_w; i++)
    if ((y_off[i] & 3) || (ws[i]->bias && (reinterpret_cast<uintptr_t>(ws[i]->bias) & 15)))
      return set_error(CAI_ERR_INVALID, "small-batch product (register form): output offsets and biases must be 16-byte aligned");
  RaParams p{};
  p.n_seg = n_w; p.eps = eps; p.swiglu_half = swiglu_half; p.y = y; p.y_stride = y_stride; p.residual = residual;
  const int cols = (int)ws[0]->cols, nsb = cols >> 8;
  // units of 32 rows (pairs of row sets), or of 16 where that shortens the longest walk (a wave takes 2 x HH items per unit)
  int HH = 2, S = 0, n_slices = 0, gx = 0, units = 0;
  {
    int u2 = 0, u1 = 0;
    for (int i = 0; i < n_w; i++) { u2 += swiglu_half > 0 ? swiglu_half / 16 : (int)(ws[i]->rows / 32); u1 += (int)(ws[i]->rows / 16); }
    bool whole_pairs = true;
    for (int i = 0; i < n_w; i++) whole_pairs = whole_pairs && ws[i]->rows % 32 == 0;
    int S2 = 0, ns2 = 0, g2 = 0, S1 = 0, ns1 = 0, g1 = 0;
    if (!ra_geometry(nsb, u2, S2, ns2, g2) || !ra_geometry(nsb, u1, S1, ns1, g1))
      return set_error(CAI_ERR_UNSUPPORTED, "small-batch product (register form): width %d", cols);
    units = u2; S = S2; n_slices = ns2; gx = g2;
    if (swiglu_half == 0 && (!whole_pairs || (u1 + g1 - 1) / g1 < 2 * ((u2 + g2 - 1) / g2))) { HH = 1; units = u1; S = S1; n_slices = ns1; gx = g1; }
  }
  int cum = 0; int64_t width = 0;
  for (int i = 0; i < n_w; i++) {
    cum += swiglu_half > 0 ? swiglu_half / 16 : (int)(ws[i]->rows / (16 * HH));
    p.seg[i] = RaSeg{ws[i]->data, ws[i]->bias, (int)ws[i]->rows, y_off[i], cum};
    width = std::max<int64_t>(width, y_off[i] + ws[i]->rows);
  }
  p.n_slices = n_slices;
  if (n_slices > 1) {
    p.part_stride = (width + 3) / 4 * 4;
    if ((size_t)n_slices * n_tok * p.part_stride > g_ra.cap_part || !g_ra.counters)
      return set_error(CAI_ERR_STATE, "small-batch product (register form): workspace not reserved (%d slices x %d tokens x %lld)", n_slices, n_tok, (long long)p.part_stride);
    p.part = g_ra.part; p.counters = g_ra.counters;
  }
  const int nw = (S + RA_SBW - 1) / RA_SBW;
  p.timeline = timeline_next(gx * n_slices);
  const dim3 grid(gx, n_slices), block(64 * nw);
  const size_t lds = (size_t)nw * RA_WAVE_LDS;
#define RA_LAUNCH(HHv, GAINv) do { \
    static bool attr_done = false; \
    if (!attr_done) { CAI_HIP(hipFuncSetAttribute((const void*)gemm_q4k_ra<HHv, GAINv>, hipFuncAttributeMaxDynamicSharedMemorySize, RA_NW * RA_WAVE_LDS)); attr_done = true; } \
    hipLaunchKernelGGL((gemm_q4k_ra<HHv, GAINv>), grid, block, lds, ctx().stream, x, (long long)x_stride, gain, cols, n_tok, units, S, p); } while (0)
  if (HH == 2 && gain) RA_LAUNCH(2, true);
  else if (HH == 2) RA_LAUNCH(2, false);
  else if (gain) RA_LAUNCH(1, true);
  else RA_LAUNCH(1, false);
#undef RA_LAUNCH
  return CAI_OK;
}

}  // namespace cai
