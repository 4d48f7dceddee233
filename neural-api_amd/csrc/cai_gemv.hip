// Block-quantized matrix-vector / small-batch kernels for gfx950 (wave64).
//
// One wave owns R output rows and walks the reduction axis with 16-byte (128-bit) loads of packed
// quant data, one "unit" per lane per step; the activation vector is staged once per work-group in
// LDS in a unit-transposed order (16 adjacent lanes read 16 adjacent float4 -> no bank conflicts)
// and reused for all rows of the wave.  Weights are dequantized in registers, accumulation is fp32,
// and the per-row sum is reduced across the 64 lanes with DPP row shifts + row broadcasts.
//
// Semantics of the layer this implements: Out[b*NumAs + a] = act(dot(W[a], X[b]) + bias[a])
// (reference: neural/neuralvolume.pas:12127-12423, 12693-12745; fused tail neural/neural.cl:111-146).
#include "cai_internal.hpp"
#include "cai_gemv_common.hpp"
#include "cai_blocks_raw.hpp"

namespace cai {

// units per lane-step and geometry per type
template <int QT> struct QTraits;
template <> struct QTraits<CAI_Q4_K> { static constexpr int UW = 32, T = 8; };  // weights per unit, float4 per unit
template <> struct QTraits<CAI_Q4_0> { static constexpr int UW = 32, T = 8; };
template <> struct QTraits<CAI_Q8_0> { static constexpr int UW = 16, T = 4; };
template <> struct QTraits<CAI_I8ROW> { static constexpr int UW = 16, T = 4; };   // per-row int8: the Q8_0 walk with one scale per row, applied at the end
// Q6_K: 16 lanes per 210-byte super-block.  Lane t (half nh = t>>3, byte position l4 = 4*(t&7)) takes four bytes each of the
// two ql runs and of the qh run of its half, i.e. the 16 weights 128*nh + 32*j + l4 + {0..3}, j = 0..3, which fall in four
// different 16-weight scale groups (neural/neuralgguf.pas:639-717).  Resident form: 192-byte ql | qh records, a plane of
// scales (16 per block) and a plane of d, all aligned.
template <> struct QTraits<CAI_Q6_K> { static constexpr int UW = 16, T = 4; };

// original float4 index n (within the panel) -> LDS float4 slot, unit-transposed in tiles of 16 units
template <int QT> __device__ __forceinline__ int lds_slot(int n)
{
  int u, t;
  if (QT == CAI_Q4_K) {
    // n = [sb][cc:2][hi:1][h:1][tt:2]; unit = sb*8 + cc*2 + h; t = hi*4 + tt
    const int sb = n >> 6, cc = (n >> 4) & 3, hi = (n >> 3) & 1, h = (n >> 2) & 1, tt = n & 3;
    u = sb * 8 + cc * 2 + h; t = hi * 4 + tt;
  } else if (QT == CAI_Q4_0) { u = n >> 3; t = n & 7; }
  else if (QT == CAI_Q6_K) { u = (n >> 6) * 16 + ((n >> 5) & 1) * 8 + (n & 7); t = (n >> 3) & 3; }   // n = [sb][nh:1][j:2][t&7:3]
  else { u = n >> 2; t = n & 3; }
  constexpr int T = QTraits<QT>::T;
  return (u >> 4) * 16 * T + t * 16 + (u & 15);
}

template <int QT> __device__ __forceinline__ int lds_unit_base(int u)
{
  constexpr int T = QTraits<QT>::T;
  return (u >> 4) * 16 * T + (u & 15);   // + t*16
}

// The four code dwords of a Q6_K lane: cj[j] holds the 6-bit codes (0..63) of weights 32*j + l4 + {0..3} of the half, one per
// byte: low nibbles from ql (j = 0, 1) or its high nibbles (j = 2, 3), bits 4..5 from the 2-bit field j of the qh bytes.
__device__ __forceinline__ void q6k_codes(uint32_t ql0, uint32_t ql1, uint32_t qh, uint32_t cj[4])
{
  cj[0] = (ql0 & 0x0f0f0f0fu) | ((qh << 4) & 0x30303030u);
  cj[1] = (ql1 & 0x0f0f0f0fu) | ((qh << 2) & 0x30303030u);
  cj[2] = ((ql0 >> 4) & 0x0f0f0f0fu) | (qh & 0x30303030u);
  cj[3] = ((ql1 >> 4) & 0x0f0f0f0fu) | ((qh >> 2) & 0x30303030u);
}

// ------------------------------------------------------------------------------------------
// Fast kernel: Q4_K / Q4_0 / Q8_0 / per-row int8.  MODE 0: plain rows.  MODE 1: SwiGLU pairs (row i and row half+i).
// ------------------------------------------------------------------------------------------
template <int QT, int NB, int R, int MODE>
__global__ __launch_bounds__(256) void gemv_fast(const GemvParams p)
{
  extern __shared__ float4 xs4[];          // [NB][kp/4]
  const unsigned long long tl0 = timeline_now();
  constexpr int UW = QTraits<QT>::UW, T = QTraits<QT>::T;
  constexpr int RR = MODE == 1 ? 2 * R : R;  // weight rows per wave
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = blockIdx.x * 4 + wave;

  // segment lookup (groups never straddle segments)
  int s = 0, grp0 = 0;
  if (p.n_seg > 1 && grp >= p.seg[0].grp_end) { s = 1; grp0 = p.seg[0].grp_end; }
  if (p.n_seg > 2 && grp >= p.seg[1].grp_end) { s = 2; grp0 = p.seg[1].grp_end; }
  const GemvSeg sg = p.seg[s];
  const int row_first = (grp - grp0) * R;
  const bool wave_live = grp < p.seg[p.n_seg - 1].grp_end;
  int64_t bank_row = 0;
  const float* xin = p.x; float* yout = p.y;
  if (p.slot_expert) {
    bank_row = (int64_t)min(max(p.slot_expert[blockIdx.y], 0), p.bank_experts - 1) * p.expert_rows;   // an id outside the bank (a router fed NaN) must not address memory
    xin += (int64_t)blockIdx.y * p.x_slot_stride; yout += (int64_t)blockIdx.y * p.y_slot_stride;
  }

  const int cols = p.cols;
  int64_t row_bytes, aux_row_bytes = 0;
  if (QT == CAI_Q4_K) row_bytes = (int64_t)(cols >> 8) * 144;
  else if (QT == CAI_Q6_K) { row_bytes = (int64_t)(cols >> 8) * 192; aux_row_bytes = (cols >> 8) * 16; }
  else if (QT == CAI_Q4_0) { row_bytes = cols >> 1; aux_row_bytes = (cols >> 5) * 2; }
  else if (QT == CAI_I8ROW) row_bytes = cols;
  else { row_bytes = cols; aux_row_bytes = (cols >> 5) * 2; }

  const uint8_t* rp[RR]; const uint8_t* ap[RR]; const uint8_t* dp[RR]; bool live[RR];
#pragma unroll
  for (int r = 0; r < RR; r++) {
    int row = row_first + (MODE == 1 ? (r >> 1) : r);
    live[r] = wave_live && row < (MODE == 1 ? p.half : sg.rows);
    if (!live[r]) row = 0;
    if (MODE == 1 && (r & 1)) row += p.half;
    rp[r] = sg.data + (bank_row + row) * row_bytes;
    ap[r] = sg.aux + (bank_row + row) * aux_row_bytes;
    dp[r] = QT == CAI_Q6_K ? p.seg_aux2[s] + (bank_row + row) * (int64_t)(cols >> 8) * 2 : nullptr;
  }

  float acc[RR][NB];
#pragma unroll
  for (int r = 0; r < RR; r++)
#pragma unroll
    for (int b = 0; b < NB; b++) acc[r][b] = 0.0f;

  // fused RMSNorm statistics (neural/neural.cl:1047-1085): inv = 1/sqrt(mean(x^2)+eps), per batch row
  float inv_rms[NB];
  if (p.norm_gain) {
    __shared__ float red[NB][4];
#pragma unroll
    for (int b = 0; b < NB; b++) {
      float ss = 0.0f;
      const float* xb = xin + (int64_t)b * cols;
      // eight requests go out before the first square is added (a request per turn would cost a cache round trip per 256
      // columns); the additions keep their order
      for (int i0 = threadIdx.x; i0 < cols; i0 += 8 * 256) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) t[u] = xb[min(i0 + u * 256, cols - 1)];
#pragma unroll
        for (int u = 0; u < 8; u++) if (i0 + u * 256 < cols) ss = fmaf(t[u], t[u], ss);
      }
      ss = wave_sum(ss);
      if (lane == 63) red[b][wave] = ss;
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < NB; b++) {
      const float tot = (red[b][0] + red[b][1]) + (red[b][2] + red[b][3]);
      inv_rms[b] = 1.0f / sqrtf(tot / (float)cols + p.norm_eps);
    }
  }

  for (int k0 = 0; k0 < cols; k0 += p.kp) {
    const int kp = min(p.kp, cols - k0);
    const int n4 = kp >> 2;
    __syncthreads();
#pragma unroll
    for (int b = 0; b < NB; b++) {
      const float4* src = reinterpret_cast<const float4*>(xin + (int64_t)b * cols + k0);
      float4* dst = xs4 + b * (p.kp_lds >> 2);
      for (int n0 = threadIdx.x; n0 < n4; n0 += 4 * 256) {     // four requests (and their gains) per turn, then the stores
        float4 v[4], g[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const int n = min(n0 + u * 256, n4 - 1);
          v[u] = src[n];
          if (p.norm_gain) g[u] = reinterpret_cast<const float4*>(p.norm_gain + k0)[n];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const int n = n0 + u * 256;
          if (n < n4) {
            float4 w = v[u];
            if (p.norm_gain) {
              w.x = g[u].x * (w.x * inv_rms[b]); w.y = g[u].y * (w.y * inv_rms[b]);
              w.z = g[u].z * (w.z * inv_rms[b]); w.w = g[u].w * (w.w * inv_rms[b]);
            }
            dst[lds_slot<QT>(n)] = w;
          }
        }
      }
    }
    __syncthreads();
    if (k0 == 0) { timeline_put(p.timeline, 0, tl0); timeline_stamp(p.timeline, 4); }

    const int n_units = kp / UW;
    for (int u = lane; u < n_units; u += 64) {
      // ---- issue all weight loads of this step first ----
      uint4 q[RR]; uint4 hdr[RR]; uint16_t dh[RR];
      if (QT == CAI_Q4_K) {
        const int sb = (k0 >> 8) + (u >> 3), j = u & 7;
#pragma unroll
        for (int r = 0; r < RR; r++) {
          const uint8_t* blk = rp[r] + (int64_t)sb * 144;
          hdr[r] = *reinterpret_cast<const uint4*>(blk);
          q[r] = *reinterpret_cast<const uint4*>(blk + 16 + 16 * j);
        }
      } else if (QT == CAI_Q6_K) {
        const int sb = (k0 >> 8) + (u >> 4), nh = (u >> 3) & 1, l4 = (u & 7) * 4;
#pragma unroll
        for (int r = 0; r < RR; r++) {
          const uint8_t* blk = rp[r] + (int64_t)sb * 192;
          q[r].x = *reinterpret_cast<const uint32_t*>(blk + 64 * nh + l4);
          q[r].y = *reinterpret_cast<const uint32_t*>(blk + 64 * nh + 32 + l4);
          q[r].z = *reinterpret_cast<const uint32_t*>(blk + 128 + 32 * nh + l4); q[r].w = 0u;
          const uint2 sc2 = *reinterpret_cast<const uint2*>(ap[r] + sb * 16 + 8 * nh);
          hdr[r].x = sc2.x; hdr[r].y = sc2.y;
          dh[r] = *reinterpret_cast<const uint16_t*>(dp[r] + sb * 2);
        }
      } else if (QT == CAI_Q4_0) {
        const int blk = (k0 >> 5) + u;
#pragma unroll
        for (int r = 0; r < RR; r++) {
          q[r] = *reinterpret_cast<const uint4*>(rp[r] + (int64_t)blk * 16);
          dh[r] = *reinterpret_cast<const uint16_t*>(ap[r] + blk * 2);
        }
      } else {
        const int un = (k0 >> 4) + u;
#pragma unroll
        for (int r = 0; r < RR; r++) {
          q[r] = *reinterpret_cast<const uint4*>(rp[r] + (int64_t)un * 16);
          dh[r] = QT == CAI_I8ROW ? (uint16_t)0x3C00 : *reinterpret_cast<const uint16_t*>(ap[r] + (un >> 1) * 2);   // per-row int8: block scale 1
        }
      }
      const int xb0 = lds_unit_base<QT>(u);

      if (NB == 1) {
        // x unit in registers, reused for every row of the wave
        float xv[UW];
#pragma unroll
        for (int t = 0; t < T; t++) {
          const float4 v = xs4[xb0 + t * 16];
          xv[4 * t] = v.x; xv[4 * t + 1] = v.y; xv[4 * t + 2] = v.z; xv[4 * t + 3] = v.w;
        }
        if (QT == CAI_Q4_K) {
          float sxlo = 0.0f, sxhi = 0.0f;
#pragma unroll
          for (int i = 0; i < 16; i++) { sxlo += xv[i]; sxhi += xv[16 + i]; }
          const int cc = (u & 7) >> 1;
#pragma unroll
          for (int r = 0; r < RR; r++) {
            const uint32_t qw[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
            float slo = 0.0f, shi = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; w++) {
              const uint32_t lo = qw[w] & 0x0f0f0f0fu, hi = (qw[w] >> 4) & 0x0f0f0f0fu;
              slo = fmaf(cvt_ub0(lo), xv[4 * w], slo);     slo = fmaf(cvt_ub1(lo), xv[4 * w + 1], slo);
              slo = fmaf(cvt_ub2(lo), xv[4 * w + 2], slo); slo = fmaf(cvt_ub3(lo), xv[4 * w + 3], slo);
              shi = fmaf(cvt_ub0(hi), xv[16 + 4 * w], shi);     shi = fmaf(cvt_ub1(hi), xv[16 + 4 * w + 1], shi);
              shi = fmaf(cvt_ub2(hi), xv[16 + 4 * w + 2], shi); shi = fmaf(cvt_ub3(hi), xv[16 + 4 * w + 3], shi);
            }
            uint32_t sc, mn; q4k_scale_pair(hdr[r].y, hdr[r].z, hdr[r].w, cc, sc, mn);
            const float d = __half2float(__ushort_as_half((unsigned short)(hdr[r].x & 0xffffu)));
            const float dmin = __half2float(__ushort_as_half((unsigned short)(hdr[r].x >> 16)));
            const float part = d * (cvt_ub0(sc) * slo + cvt_ub1(sc) * shi) - dmin * (cvt_ub0(mn) * sxlo + cvt_ub1(mn) * sxhi);
            acc[r][0] += part;
          }
        } else if (QT == CAI_Q6_K) {
          float sx[4];
#pragma unroll
          for (int j = 0; j < 4; j++) sx[j] = (xv[4 * j] + xv[4 * j + 1]) + (xv[4 * j + 2] + xv[4 * j + 3]);
          const int hs = (u & 4) ? 8 : 0;    // positions 16..31 of a 32-run use the odd scale of the pair
#pragma unroll
          for (int r = 0; r < RR; r++) {
            uint32_t cj[4]; q6k_codes(q[r].x, q[r].y, q[r].z, cj);
            const uint32_t s01 = hdr[r].x >> hs, s23 = hdr[r].y >> hs;
            const float sc[4] = {(float)(int8_t)(s01 & 0xff), (float)(int8_t)((s01 >> 16) & 0xff), (float)(int8_t)(s23 & 0xff), (float)(int8_t)((s23 >> 16) & 0xff)};
            float part = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
              float sq = cvt_ub0(cj[j]) * xv[4 * j];
              sq = fmaf(cvt_ub1(cj[j]), xv[4 * j + 1], sq); sq = fmaf(cvt_ub2(cj[j]), xv[4 * j + 2], sq); sq = fmaf(cvt_ub3(cj[j]), xv[4 * j + 3], sq);
              part = fmaf(sc[j], fmaf(-32.0f, sx[j], sq), part);
            }
            acc[r][0] = fmaf(__half2float(__ushort_as_half(dh[r])), part, acc[r][0]);
          }
        } else if (QT == CAI_Q4_0) {
          float sx = 0.0f;
#pragma unroll
          for (int i = 0; i < 32; i++) sx += xv[i];
#pragma unroll
          for (int r = 0; r < RR; r++) {
            const uint32_t qw[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
            float sq = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; w++) {
              const uint32_t lo = qw[w] & 0x0f0f0f0fu, hi = (qw[w] >> 4) & 0x0f0f0f0fu;
              sq = fmaf(cvt_ub0(lo), xv[4 * w], sq);     sq = fmaf(cvt_ub1(lo), xv[4 * w + 1], sq);
              sq = fmaf(cvt_ub2(lo), xv[4 * w + 2], sq); sq = fmaf(cvt_ub3(lo), xv[4 * w + 3], sq);
              sq = fmaf(cvt_ub0(hi), xv[16 + 4 * w], sq);     sq = fmaf(cvt_ub1(hi), xv[16 + 4 * w + 1], sq);
              sq = fmaf(cvt_ub2(hi), xv[16 + 4 * w + 2], sq); sq = fmaf(cvt_ub3(hi), xv[16 + 4 * w + 3], sq);
            }
            const float d = __half2float(__ushort_as_half(dh[r]));
            acc[r][0] = fmaf(d, sq - 8.0f * sx, acc[r][0]);
          }
        } else {  // Q8_0
#pragma unroll
          for (int r = 0; r < RR; r++) {
            const uint32_t qw[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
            float sq = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; w++) {
              sq = fmaf((float)(int8_t)(qw[w] & 0xff), xv[4 * w], sq);
              sq = fmaf((float)(int8_t)((qw[w] >> 8) & 0xff), xv[4 * w + 1], sq);
              sq = fmaf((float)(int8_t)((qw[w] >> 16) & 0xff), xv[4 * w + 2], sq);
              sq = fmaf((float)(int8_t)(qw[w] >> 24), xv[4 * w + 3], sq);
            }
            acc[r][0] = fmaf(__half2float(__ushort_as_half(dh[r])), sq, acc[r][0]);
          }
        }
      } else {
        // small batch: dequantize the unit of every row once (unscaled integer values as floats),
        // then stream the NB activation units from LDS
        float wf[RR][UW];
        float s0[RR], s1[RR], m0[RR], m1[RR];
#pragma unroll
        for (int r = 0; r < RR; r++) {
          const uint32_t qw[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
          if (QT == CAI_Q6_K) {
            uint32_t cj[4]; q6k_codes(q[r].x, q[r].y, q[r].z, cj);
            const int hs = (u & 4) ? 8 : 0;
            const uint32_t s01 = hdr[r].x >> hs, s23 = hdr[r].y >> hs;
            const float d = __half2float(__ushort_as_half(dh[r]));
            // the four group scales of the lane travel in s0, s1, m0, m1
            s0[r] = d * (float)(int8_t)(s01 & 0xff); s1[r] = d * (float)(int8_t)((s01 >> 16) & 0xff);
            m0[r] = d * (float)(int8_t)(s23 & 0xff); m1[r] = d * (float)(int8_t)((s23 >> 16) & 0xff);
#pragma unroll
            for (int j = 0; j < 4; j++) {
              wf[r][4 * j] = cvt_ub0(cj[j]) - 32.0f; wf[r][4 * j + 1] = cvt_ub1(cj[j]) - 32.0f;
              wf[r][4 * j + 2] = cvt_ub2(cj[j]) - 32.0f; wf[r][4 * j + 3] = cvt_ub3(cj[j]) - 32.0f;
            }
          } else if (QT == CAI_Q8_0 || QT == CAI_I8ROW) {
#pragma unroll
            for (int w = 0; w < 4; w++) {
              wf[r][4 * w] = (float)(int8_t)(qw[w] & 0xff); wf[r][4 * w + 1] = (float)(int8_t)((qw[w] >> 8) & 0xff);
              wf[r][4 * w + 2] = (float)(int8_t)((qw[w] >> 16) & 0xff); wf[r][4 * w + 3] = (float)(int8_t)(qw[w] >> 24);
            }
            s0[r] = __half2float(__ushort_as_half(dh[r]));
          } else {
#pragma unroll
            for (int w = 0; w < 4; w++) {
              const uint32_t lo = qw[w] & 0x0f0f0f0fu, hi = (qw[w] >> 4) & 0x0f0f0f0fu;
              wf[r][4 * w] = cvt_ub0(lo); wf[r][4 * w + 1] = cvt_ub1(lo); wf[r][4 * w + 2] = cvt_ub2(lo); wf[r][4 * w + 3] = cvt_ub3(lo);
              wf[r][16 + 4 * w] = cvt_ub0(hi); wf[r][16 + 4 * w + 1] = cvt_ub1(hi); wf[r][16 + 4 * w + 2] = cvt_ub2(hi); wf[r][16 + 4 * w + 3] = cvt_ub3(hi);
            }
            if (QT == CAI_Q4_K) {
              uint32_t sc, mn; q4k_scale_pair(hdr[r].y, hdr[r].z, hdr[r].w, (u & 7) >> 1, sc, mn);
              const float d = __half2float(__ushort_as_half((unsigned short)(hdr[r].x & 0xffffu)));
              const float dmin = __half2float(__ushort_as_half((unsigned short)(hdr[r].x >> 16)));
              s0[r] = d * cvt_ub0(sc); s1[r] = d * cvt_ub1(sc); m0[r] = dmin * cvt_ub0(mn); m1[r] = dmin * cvt_ub1(mn);
            } else s0[r] = __half2float(__ushort_as_half(dh[r]));
          }
        }
#pragma unroll
        for (int b = 0; b < NB; b++) {
          float xv[UW];
          const float4* xb = xs4 + b * (p.kp_lds >> 2);
#pragma unroll
          for (int t = 0; t < T; t++) {
            const float4 v = xb[xb0 + t * 16];
            xv[4 * t] = v.x; xv[4 * t + 1] = v.y; xv[4 * t + 2] = v.z; xv[4 * t + 3] = v.w;
          }
          if (QT == CAI_Q6_K) {
#pragma unroll
            for (int r = 0; r < RR; r++) {
              float g[4];
#pragma unroll
              for (int j = 0; j < 4; j++) {
                g[j] = wf[r][4 * j] * xv[4 * j];
                g[j] = fmaf(wf[r][4 * j + 1], xv[4 * j + 1], g[j]); g[j] = fmaf(wf[r][4 * j + 2], xv[4 * j + 2], g[j]); g[j] = fmaf(wf[r][4 * j + 3], xv[4 * j + 3], g[j]);
              }
              acc[r][b] += (s0[r] * g[0] + s1[r] * g[1]) + (m0[r] * g[2] + m1[r] * g[3]);
            }
          } else if (QT == CAI_Q8_0 || QT == CAI_I8ROW) {
#pragma unroll
            for (int r = 0; r < RR; r++) {
              float sq = 0.0f;
#pragma unroll
              for (int i = 0; i < 16; i++) sq = fmaf(wf[r][i], xv[i], sq);
              acc[r][b] = fmaf(s0[r], sq, acc[r][b]);
            }
          } else if (QT == CAI_Q4_0) {
            float sx = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; i++) sx += xv[i];
#pragma unroll
            for (int r = 0; r < RR; r++) {
              float sq = 0.0f;
#pragma unroll
              for (int i = 0; i < 32; i++) sq = fmaf(wf[r][i], xv[i], sq);
              acc[r][b] = fmaf(s0[r], sq - 8.0f * sx, acc[r][b]);
            }
          } else {
            float sxlo = 0.0f, sxhi = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; i++) { sxlo += xv[i]; sxhi += xv[16 + i]; }
#pragma unroll
            for (int r = 0; r < RR; r++) {
              float slo = 0.0f, shi = 0.0f;
#pragma unroll
              for (int i = 0; i < 16; i++) { slo = fmaf(wf[r][i], xv[i], slo); shi = fmaf(wf[r][16 + i], xv[16 + i], shi); }
              acc[r][b] += (s0[r] * slo + s1[r] * shi) - (m0[r] * sxlo + m1[r] * sxhi);
            }
          }
        }
      }
    }
  }

  // ---- reduce across the wave and write ----
  timeline_stamp(p.timeline, 5);
#pragma unroll
  for (int r = 0; r < RR; r++)
#pragma unroll
    for (int b = 0; b < NB; b++) acc[r][b] = wave_sum(acc[r][b]);

  if (lane == 63) {
    if (MODE == 0) {
#pragma unroll
      for (int r = 0; r < RR; r++) {
        if (!live[r]) continue;
        const int row = row_first + r;
#pragma unroll
        for (int b = 0; b < NB; b++) {
          float v = acc[r][b];
          if (QT == CAI_I8ROW) v *= reinterpret_cast<const float*>(sg.aux)[bank_row + row];   // (sum code * x) * scale, then bias (neural/neuralvolume.pas:12693-12745)
          if (sg.bias) v += sg.bias[bank_row + row];
          v = act_apply(v, p.act);
          const int64_t o = (int64_t)b * p.y_stride + sg.y_off + row;
          if (p.residual) v += p.residual[o];
          yout[o] = v;
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; r++) {
        if (!live[2 * r]) continue;
        const int row = row_first + r;
#pragma unroll
        for (int b = 0; b < NB; b++) {
          float up = acc[2 * r][b], gate = acc[2 * r + 1][b];
          if (sg.bias) { up += sg.bias[bank_row + row]; gate += sg.bias[bank_row + p.half + row]; }
          yout[(int64_t)b * p.y_stride + sg.y_off + row] = silu_mul(up, gate);
        }
      }
    }
  }
  timeline_stamp(p.timeline, 7);
}

// ------------------------------------------------------------------------------------------
// Simple kernel: F32 / F16 and the per-row int8 widths the fast kernel does not take.  One wave per row,
// lanes stride the row with scalar loads (coalesced), fp32 accumulation.
// ------------------------------------------------------------------------------------------
template <int QT>
__global__ __launch_bounds__(256) void gemv_simple(const GemvParams p, int n_b)
{
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t grow = (int64_t)blockIdx.x * 4 + wave;
  int s = 0; int64_t g0 = 0;
  if (p.n_seg > 1 && grow >= p.seg[0].grp_end) { s = 1; g0 = p.seg[0].grp_end; }
  if (p.n_seg > 2 && grow >= p.seg[1].grp_end) { s = 2; g0 = p.seg[1].grp_end; }
  if (grow >= p.seg[p.n_seg - 1].grp_end) return;
  const GemvSeg sg = p.seg[s];
  const int row = (int)(grow - g0);
  const int cols = p.cols;
  int64_t bank_row = 0;
  const float* xin = p.x; float* yout = p.y;
  if (p.slot_expert) {
    bank_row = (int64_t)min(max(p.slot_expert[blockIdx.y], 0), p.bank_experts - 1) * p.expert_rows;   // an id outside the bank (a router fed NaN) must not address memory
    xin += (int64_t)blockIdx.y * p.x_slot_stride; yout += (int64_t)blockIdx.y * p.y_slot_stride;
  }
  const int64_t wrow = bank_row + row;
  for (int b = 0; b < n_b; b++) {
    const float* xb = xin + (int64_t)b * cols;
    float inv = 1.0f;
    if (p.norm_gain) {
      float ss = 0.0f;
      for (int i = lane; i < cols; i += 64) ss = fmaf(xb[i], xb[i], ss);
      ss = wave_sum(ss);
      ss = __shfl(ss, 63);
      inv = 1.0f / sqrtf(ss / (float)cols + p.norm_eps);
    }
    float acc = 0.0f;
    for (int i = lane; i < cols; i += 64) {
      float w;
      if (QT == CAI_F32) w = reinterpret_cast<const float*>(sg.data)[wrow * cols + i];
      else if (QT == CAI_F16) w = __half2float(reinterpret_cast<const __half*>(sg.data)[wrow * cols + i]);
      else w = (float)reinterpret_cast<const int8_t*>(sg.data)[wrow * cols + i];
      float xv = xb[i];
      if (p.norm_gain) xv = p.norm_gain[i] * (xv * inv);
      acc = fmaf(w, xv, acc);
    }
    acc = wave_sum(acc);
    if (lane == 63) {
      if (QT == CAI_I8ROW) acc *= reinterpret_cast<const float*>(sg.aux)[wrow];
      if (sg.bias) acc += sg.bias[wrow];
      acc = act_apply(acc, p.act);
      const int64_t o = (int64_t)b * p.y_stride + sg.y_off + row;
      if (p.residual) acc += p.residual[o];
      yout[o] = acc;
    }
  }
}

// ------------------------------------------------------------------------------------------
// Block types resident as the stored stream (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K).  A wave takes four consecutive rows; a
// lane decodes runs of 16 consecutive weights (run = lane + 64 k, so the 16 lanes of a super-block share its header in
// cache).  The activation values of a run are fetched once for the four rows (one row per wave moved six times the
// weight bytes through the vector cache), and one decode feeds every batch row.  fp32 accumulation; fused RMSNorm, bias,
// activation, residual and the expert-bank gather as in the other kernels.
// ------------------------------------------------------------------------------------------
template <int QT, int NB>   // NB: batch rows the accumulators cover (1 or 8)
__global__ __launch_bounds__(256) void gemv_raw(const GemvParams p, int n_b)
{
  constexpr int R = 4;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t grp = (int64_t)blockIdx.x * 4 + wave;
  int s = 0; int64_t g0 = 0;
  if (p.n_seg > 1 && grp >= p.seg[0].grp_end) { s = 1; g0 = p.seg[0].grp_end; }
  if (p.n_seg > 2 && grp >= p.seg[1].grp_end) { s = 2; g0 = p.seg[1].grp_end; }
  if (grp >= p.seg[p.n_seg - 1].grp_end) return;
  const GemvSeg sg = p.seg[s];
  const int row0 = (int)(grp - g0) * R;
  const int cols = p.cols;
  int64_t bank_row = 0;
  const float* xin = p.x; float* yout = p.y;
  if (p.slot_expert) {
    bank_row = (int64_t)min(max(p.slot_expert[blockIdx.y], 0), p.bank_experts - 1) * p.expert_rows;
    xin += (int64_t)blockIdx.y * p.x_slot_stride; yout += (int64_t)blockIdx.y * p.y_slot_stride;
  }
  const int64_t row_bytes = (int64_t)(cols / raw_block_elems(QT)) * raw_block_bytes(QT);
  const uint8_t* wbase[R];
#pragma unroll
  for (int r = 0; r < R; r++) wbase[r] = sg.data + (bank_row + min(row0 + r, sg.rows - 1)) * row_bytes;   // tail group: the last row again, not written
  float inv[NB];
#pragma unroll
  for (int b = 0; b < NB; b++) {
    inv[b] = 1.0f;
    if (p.norm_gain && b < n_b) {
      const float* xb = xin + (int64_t)b * cols;
      float ss = 0.0f;
      for (int i = lane * 4; i < cols; i += 256) { const float4 v = *reinterpret_cast<const float4*>(xb + i); ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss); }
      ss = __shfl(wave_sum(ss), 63);
      inv[b] = 1.0f / sqrtf(ss / (float)cols + p.norm_eps);
    }
  }
  float acc[R][NB];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int b = 0; b < NB; b++) acc[r][b] = 0.0f;
  const int n_runs = cols >> 4;
  for (int run = lane; run < n_runs; run += 64) {
    float w[R][16];
#pragma unroll
    for (int r = 0; r < R; r++) raw_run16<QT>(wbase[r], run, w[r]);
    float g[16];
    if (p.norm_gain) {
#pragma unroll
      for (int q = 0; q < 4; q++) { const float4 v = *reinterpret_cast<const float4*>(p.norm_gain + 16 * run + 4 * q); g[4 * q] = v.x; g[4 * q + 1] = v.y; g[4 * q + 2] = v.z; g[4 * q + 3] = v.w; }
    }
#pragma unroll
    for (int b = 0; b < NB; b++) {
      if (b < n_b) {
        const float* xb = xin + (int64_t)b * cols + 16 * run;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const float4 v = *reinterpret_cast<const float4*>(xb + 4 * q);
          const float xv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int t = 0; t < 4; t++) {
            const float xn = p.norm_gain ? g[4 * q + t] * (xv[t] * inv[b]) : xv[t];
#pragma unroll
            for (int r = 0; r < R; r++) acc[r][b] = fmaf(w[r][4 * q + t], xn, acc[r][b]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int b = 0; b < NB; b++) {
      if (b < n_b) {
        float a = wave_sum(acc[r][b]);
        const int row = row0 + r;
        if (lane == 63 && row < sg.rows) {
          if (sg.bias) a += sg.bias[bank_row + row];
          a = act_apply(a, p.act);
          const int64_t o = (int64_t)b * p.y_stride + sg.y_off + row;
          if (p.residual) a += p.residual[o];
          yout[o] = a;
        }
      }
    }
}

// y[b][i] = x[b][i] * silu(x[b][half+i]) for the simple path (unfused SwiGLU)
__global__ void swiglu_rows(const float* x, int half, int n_tokens, float* y)
{
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)half * n_tokens) return;
  const int t = (int)(i / half), d = (int)(i - (int64_t)t * half);
  y[i] = silu_mul(x[(int64_t)t * 2 * half + d], x[(int64_t)t * 2 * half + half + d]);
}

int launch_q4k_dot(GemvParams& p, const MultiGemv& m, int swiglu_half, hipStream_t st);
// True when a batch-1 launch on this matrix goes through the streaming kernel (which honours ssq_in / ssq_out).
bool gemv_hands_off_ssq(const cai_qw_s* w, int n_b)
{
  return (w->qtype == CAI_Q4_K || w->qtype == CAI_Q5_K) && n_b == 1 && w->cols % 256 == 0 && (((w->cols >> 8) + 15) >> 4) <= 8;
}
// True when launch_gemv_multi takes this matrix with the SwiGLU epilogue (swiglu_half != 0) at this batch width.
bool gemv_fuses_swiglu(const cai_qw_s* w, int n_b, bool expert_bank)
{
  if (w->qtype == CAI_Q4_K || w->qtype == CAI_Q4_0 || w->qtype == CAI_Q8_0) return true;
  return w->qtype == CAI_Q5_K && n_b == 1 && !expert_bank && gemv_hands_off_ssq(w, 1);   // (integer-dot kernel only)
}
static bool fast_type(int qt) { return qt == CAI_Q4_K || qt == CAI_Q4_0 || qt == CAI_Q8_0; }

static int panel_len(int cols, int nb)
{
  int kp = 8192;
  while ((int64_t)kp * nb * 4 > 65536) kp >>= 1;
  const int cols256 = (cols + 255) / 256 * 256;
  if (kp > cols256) kp = cols256;
  return kp;
}

template <int QT, int NB, int MODE>
static int launch_fast_r(const GemvParams& p0, int n_groups_r, int R, int n_slots, hipStream_t st)
{
  GemvParams p = p0;
  const size_t lds = (size_t)NB * p.kp_lds * 4;
  const dim3 grid((n_groups_r + 3) / 4, n_slots);
  p.timeline = timeline_next((int)(grid.x * grid.y));
  if constexpr (NB == 1 && MODE == 0) {
    if (R == 4) { hipLaunchKernelGGL((gemv_fast<QT, NB, 4, MODE>), grid, dim3(256), lds, st, p); return CAI_OK; }
  }
  if (R == 4) return set_error(CAI_ERR_INVALID, "gemv: 4 rows per wave only exists for batch 1 plain rows");
  if (R == 2) hipLaunchKernelGGL((gemv_fast<QT, NB, 2, MODE>), grid, dim3(256), lds, st, p);
  else hipLaunchKernelGGL((gemv_fast<QT, NB, 1, MODE>), grid, dim3(256), lds, st, p);
  return CAI_OK;
}

// Rows per wave: enough groups to give every CU several waves, more rows per wave when the matrix is tall.
static int pick_r(int64_t total_rows, int nb, int mode)
{
  if (nb > 1 || mode == 1) return total_rows >= 16384 ? 2 : 1;
  if (total_rows >= 32768) return 4;
  if (total_rows >= 8192) return 2;
  return 1;
}


template <int QT, int MODE>
static int launch_fast_nb(GemvParams& p, const MultiGemv& m, int nb, hipStream_t st)
{
  int64_t total = 0;
  for (int i = 0; i < m.n; i++) total += m.rows[i];
  const int ns = m.slot_expert ? m.n_slots : 1;
  const int R = pick_r((MODE == 1 ? 2 * total : total) * ns, nb, MODE);
  int cum = 0;
  for (int i = 0; i < m.n; i++) {
    cum += (int)((m.rows[i] + R - 1) / R);
    p.seg[i].grp_end = cum;
  }
  switch (nb) {
    case 1: return launch_fast_r<QT, 1, MODE>(p, cum, R, ns, st);
    case 2: return launch_fast_r<QT, 2, MODE>(p, cum, R, ns, st);
    case 3: return launch_fast_r<QT, 3, MODE>(p, cum, R, ns, st);
    case 4: return launch_fast_r<QT, 4, MODE>(p, cum, R, ns, st);
    case 5: return launch_fast_r<QT, 5, MODE>(p, cum, R, ns, st);
    case 6: return launch_fast_r<QT, 6, MODE>(p, cum, R, ns, st);
    case 7: return launch_fast_r<QT, 7, MODE>(p, cum, R, ns, st);
    case 8: return launch_fast_r<QT, 8, MODE>(p, cum, R, ns, st);
  }
  return set_error(CAI_ERR_INVALID, "gemv: n_b %d out of range 1..8", nb);
}

static int64_t data_row_bytes(const cai_qw_s* w)
{
  switch (w->qtype) {
    case CAI_Q4_K: return w->cols / 256 * 144;
    case CAI_Q6_K: return w->cols / 256 * 192;
    case CAI_Q4_0: return w->cols / 2;
    case CAI_Q8_0: case CAI_I8ROW: return w->cols;
    case CAI_F32: return w->cols * 4;
    case CAI_F16: return w->cols * 2;
  }
  if (raw_block_type(w->qtype)) return w->cols / raw_block_elems(w->qtype) * raw_block_bytes(w->qtype);
  return 0;
}
static int64_t aux_row_bytes(const cai_qw_s* w)
{
  if (w->qtype == CAI_Q4_0 || w->qtype == CAI_Q8_0) return w->cols / 32 * 2;
  if (w->qtype == CAI_I8ROW) return 4;
  if (w->qtype == CAI_Q6_K) return w->cols / 256 * 16;
  return 0;
}

// Up to three matrices of one type and width share the staged activation (q|k|v in one launch).
int launch_gemv_multi(const MultiGemv& m, const float* x, int n_b, float* y, int64_t y_stride, int act,
                      const float* residual, const float* norm_gain, float norm_eps, int swiglu_half)
{
  Context& c = ctx();
  const cai_qw_s* w0 = m.w[0];
  GemvParams p{};
  p.n_seg = m.n; p.x = x; p.y = y; p.residual = residual; p.norm_gain = norm_gain; p.norm_eps = norm_eps;
  p.cols = (int)w0->cols; p.y_stride = (int)y_stride; p.act = act; p.half = swiglu_half;
  p.ssq_in = nullptr; p.ssq_out = nullptr;
  p.slot_expert = m.slot_expert; p.expert_rows = m.expert_rows; p.x_slot_stride = m.x_slot_stride; p.y_slot_stride = m.y_slot_stride;
  const int n_slots = m.slot_expert ? m.n_slots : 1;
  if (m.slot_expert) {
    if (m.n != 1 || m.expert_rows <= 0 || w0->rows % m.expert_rows || m.row0[0] != 0 || m.rows[0] > m.expert_rows)
      return set_error(CAI_ERR_INVALID, "gemv: expert bank of %lld rows does not divide into windows of %lld", (long long)w0->rows, (long long)m.expert_rows);
    p.bank_experts = (int)(w0->rows / m.expert_rows);
  }
  for (int i = 0; i < m.n; i++) {
    const cai_qw_s* w = m.w[i];
    if (w->qtype != w0->qtype || w->cols != w0->cols) return set_error(CAI_ERR_INVALID, "gemv: fused matrices differ in type or width");
    if (m.row0[i] < 0 || m.rows[i] <= 0 || m.row0[i] + m.rows[i] > w->rows)
      return set_error(CAI_ERR_INVALID, "gemv: row range [%lld,+%lld) outside matrix of %lld rows", (long long)m.row0[i], (long long)m.rows[i], (long long)w->rows);
    p.seg[i].data = w->data + m.row0[i] * data_row_bytes(w);
    p.seg[i].aux = w->aux ? w->aux + m.row0[i] * aux_row_bytes(w) : nullptr;
    p.seg_aux2[i] = w->qtype == CAI_Q6_K ? qw_aux2(w) + m.row0[i] * (w->cols / 256) * 2 : nullptr;
    p.seg[i].bias = w->bias ? w->bias + m.row0[i] : nullptr;
    p.seg[i].rows = (int)m.rows[i];
    p.seg[i].y_off = m.y_off[i];
  }
  const int qt = w0->qtype;
  if ((qt == CAI_Q4_K || qt == CAI_Q5_K || (qt == CAI_Q4_0 && p.cols % 256 == 0) || (qt == CAI_Q6_K && m.n == 1 && !swiglu_half)) && n_b == 1 && !m.slot_expert) {
    MultiGemv mm = m;
    if (swiglu_half) { if (m.n != 1) return set_error(CAI_ERR_INVALID, "gemv: swiglu takes one matrix"); p.seg[0].rows = swiglu_half; }
    p.ssq_in = m.ssq_in; p.ssq_out = m.ssq_out;
    const int rc = launch_q4k_dot(p, mm, swiglu_half, c.stream);
    p.ssq_in = nullptr; p.ssq_out = nullptr;
    if (rc != CAI_ERR_UNSUPPORTED) return rc;
  }
  if (fast_type(qt)) {
    p.kp = panel_len(p.cols, n_b);
    p.kp_lds = (p.kp + 511) / 512 * 512;
    if (swiglu_half) {
      if (m.n != 1) return set_error(CAI_ERR_INVALID, "gemv: swiglu takes one matrix");
      p.seg[0].rows = swiglu_half;
      MultiGemv mm = m; mm.rows[0] = swiglu_half;
      if (qt == CAI_Q4_K) return launch_fast_nb<CAI_Q4_K, 1>(p, mm, n_b, c.stream);
      if (qt == CAI_Q4_0) return launch_fast_nb<CAI_Q4_0, 1>(p, mm, n_b, c.stream);
      return launch_fast_nb<CAI_Q8_0, 1>(p, mm, n_b, c.stream);
    }
    if (qt == CAI_Q4_K) return launch_fast_nb<CAI_Q4_K, 0>(p, m, n_b, c.stream);
    if (qt == CAI_Q4_0) return launch_fast_nb<CAI_Q4_0, 0>(p, m, n_b, c.stream);
    return launch_fast_nb<CAI_Q8_0, 0>(p, m, n_b, c.stream);
  }
  if (qt == CAI_I8ROW && p.cols % 32 == 0 && !swiglu_half) {   // per-row int8 of a width the 16-byte walk covers; other widths below
    p.kp = panel_len(p.cols, n_b);
    p.kp_lds = (p.kp + 511) / 512 * 512;
    return launch_fast_nb<CAI_I8ROW, 0>(p, m, n_b, c.stream);
  }
  if (qt == CAI_Q6_K && !swiglu_half) {
    p.kp = panel_len(p.cols, n_b);
    p.kp_lds = (p.kp + 511) / 512 * 512;
    return launch_fast_nb<CAI_Q6_K, 0>(p, m, n_b, c.stream);
  }
  if (swiglu_half) return set_error(CAI_ERR_UNSUPPORTED, "gemv: fused swiglu needs a block-quantized matrix");
  if (raw_block_type(qt)) {
    const int R = 4;
    int64_t groups = 0;
    for (int i = 0; i < m.n; i++) { groups += (m.rows[i] + R - 1) / R; p.seg[i].grp_end = (int)groups; }
    const dim3 grid((unsigned)((groups + 3) / 4), n_slots);
    auto go = [&](auto k1, auto k8) { if (n_b == 1) hipLaunchKernelGGL(k1, grid, dim3(256), 0, c.stream, p, n_b); else hipLaunchKernelGGL(k8, grid, dim3(256), 0, c.stream, p, n_b); };
    switch (qt) {
      case CAI_Q5_K: go(gemv_raw<CAI_Q5_K, 1>, gemv_raw<CAI_Q5_K, 8>); break;
      case CAI_Q2_K: go(gemv_raw<CAI_Q2_K, 1>, gemv_raw<CAI_Q2_K, 8>); break;
      case CAI_Q3_K: go(gemv_raw<CAI_Q3_K, 1>, gemv_raw<CAI_Q3_K, 8>); break;
      case CAI_Q4_1: go(gemv_raw<CAI_Q4_1, 1>, gemv_raw<CAI_Q4_1, 8>); break;
      case CAI_Q5_0: go(gemv_raw<CAI_Q5_0, 1>, gemv_raw<CAI_Q5_0, 8>); break;
      default: go(gemv_raw<CAI_Q5_1, 1>, gemv_raw<CAI_Q5_1, 8>); break;
    }
    return CAI_OK;
  }
  int64_t cum = 0;
  for (int i = 0; i < m.n; i++) { cum += m.rows[i]; p.seg[i].grp_end = (int)cum; }
  const dim3 grid((unsigned)((cum + 3) / 4), n_slots);
  if (qt == CAI_F32) hipLaunchKernelGGL(gemv_simple<CAI_F32>, grid, dim3(256), 0, c.stream, p, n_b);
  else if (qt == CAI_F16) hipLaunchKernelGGL(gemv_simple<CAI_F16>, grid, dim3(256), 0, c.stream, p, n_b);
  else if (qt == CAI_I8ROW) hipLaunchKernelGGL(gemv_simple<CAI_I8ROW>, grid, dim3(256), 0, c.stream, p, n_b);
  else return set_error(CAI_ERR_UNSUPPORTED, "gemv: weight type %d", qt);
  return CAI_OK;
}

int launch_gemv(const cai_qw_s* w, int64_t row0, int64_t n_rows, const float* x, int n_b, float* y,
                int64_t y_stride, int act, const float* residual)
{
  MultiGemv m{}; m.n = 1; m.w[0] = w; m.row0[0] = row0; m.rows[0] = n_rows; m.y_off[0] = 0;
  return launch_gemv_multi(m, x, n_b, y, y_stride, act, residual, nullptr, 0.0f, 0);
}

int launch_swiglu(const float* x, int half, int n_tokens, float* y)
{
  const int64_t n = (int64_t)half * n_tokens;
  hipLaunchKernelGGL(swiglu_rows, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx().stream, x, half, n_tokens, y);
  return CAI_OK;
}

}  // namespace cai
