// Decoders of the GGUF block types that stay resident as the stored block stream: Q4_1, Q5_0, Q5_1 (32 weights per block)
// and Q2_K, Q3_K, Q5_K (256 per super-block).  Two forms of one definition: a single element (dequantise / embedding
// gather) and a run of 16 consecutive weights (the matrix-vector kernel).  Every product of a format below is exact in
// binary32 (an 11-bit half times at most 6 + 5 bits of integer) and at most one addition rounds, so both forms return
// the bits of DecodeGGMLSpan (neural/neuralgguf.pas:1471-1523) whatever the order of evaluation.
#pragma once
#include "cai_internal.hpp"

namespace cai {

__device__ __forceinline__ float raw_half(const uint8_t* p) { return __half2float(__ushort_as_half(*reinterpret_cast<const uint16_t*>(p))); }
// 32 bits at an address that is only 2-byte aligned (22- and 110-byte blocks)
__device__ __forceinline__ uint32_t raw_u32_a2(const uint8_t* p)
{
  const uint16_t* h = reinterpret_cast<const uint16_t*>(p);
  return (uint32_t)h[0] | ((uint32_t)h[1] << 16);
}

// The packed 6-bit (scale, min) pair of sub-block j of a Q4_K / Q5_K super-block (neural/neuralgguf.pas:448-464)
__device__ __forceinline__ void k_scale_min(const uint8_t* s, int j, int& sc, int& mn)
{
  if (j < 4) { sc = s[j] & 63; mn = s[j + 4] & 63; }
  else { sc = (s[j + 4] & 15) | ((s[j - 4] >> 2) & 0x30); mn = (s[j + 4] >> 4) | ((s[j] >> 2) & 0x30); }
}
// Q3_K: signed 6-bit scale of the 16-element sub-block j from the 12 packed bytes (neural/neuralgguf.pas:738-760)
__device__ __forceinline__ int q3k_scale(const uint8_t* sp, int j)
{
  const int lo = j < 8 ? (sp[j & 7] & 15) : (sp[j & 7] >> 4);
  const int hi = (sp[8 + (j & 3)] >> (2 * (j >> 2))) & 3;
  return (lo | (hi << 4)) - 32;
}

// Element e of the block at blk.
__device__ __forceinline__ float raw_block_elem(int qt, const uint8_t* blk, int e)
{
  switch (qt) {
    case CAI_Q4_1: {  // x = d * nibble + m (neural/neuralgguf.pas:846-873)
      const uint8_t b = blk[4 + (e & 15)];
      return fmaf(raw_half(blk), (float)(e < 16 ? (b & 15) : (b >> 4)), raw_half(blk + 2));
    }
    case CAI_Q5_0: {  // x = d * ((nibble | bit e of qh << 4) - 16) (neural/neuralgguf.pas:874-908)
      const uint8_t b = blk[6 + (e & 15)];
      const int q = (e < 16 ? (b & 15) : (b >> 4)) | (int)(((raw_u32_a2(blk + 2) >> e) & 1u) << 4);
      return raw_half(blk) * (float)(q - 16);
    }
    case CAI_Q5_1: {  // x = d * (nibble | bit << 4) + m (neural/neuralgguf.pas:909-944)
      const uint8_t b = blk[8 + (e & 15)];
      const int q = (e < 16 ? (b & 15) : (b >> 4)) | (int)(((*reinterpret_cast<const uint32_t*>(blk + 4) >> e) & 1u) << 4);
      return fmaf(raw_half(blk), (float)q, raw_half(blk + 2));
    }
    case CAI_Q2_K: {  // x = (d * scale) * q - dmin * min (neural/neuralgguf.pas:588-648)
      const uint8_t scb = blk[e >> 4];
      const float dl = raw_half(blk + 80) * (float)(scb & 15), ml = raw_half(blk + 82) * (float)(scb >> 4);
      const int q = (blk[16 + (e >> 7) * 32 + (e & 31)] >> (2 * ((e & 127) >> 5))) & 3;
      return fmaf(dl, (float)q, -ml);
    }
    case CAI_Q3_K: {  // x = (d * scale) * (q - 4 when the mask bit is clear) (neural/neuralgguf.pas:718-806)
      const float dl = raw_half(blk + 108) * (float)q3k_scale(blk + 96, e >> 4);
      const int ql = (blk[32 + (e >> 7) * 32 + (e & 31)] >> (2 * ((e & 127) >> 5))) & 3;
      const int clear = ((blk[e & 31] >> (e >> 5)) & 1) ^ 1;
      return dl * (float)(ql - (clear << 2));
    }
    case CAI_Q5_K: {  // x = (d * sc) * (nibble | bit << 4) - dmin * mn (neural/neuralgguf.pas:516-587)
      const int c = e >> 6, hi = (e >> 5) & 1, i = e & 31, j = 2 * c + hi;
      int sc, mn; k_scale_min(blk + 4, j, sc, mn);
      const uint8_t b = blk[48 + 32 * c + i];
      const int q = (hi ? (b >> 4) : (b & 15)) | (((blk[16 + i] >> j) & 1) << 4);
      return fmaf(raw_half(blk) * (float)sc, (float)q, -(raw_half(blk + 2) * (float)mn));
    }
  }
  return 0.0f;
}

// 16 bytes from an address aligned to A bytes (A = 2, 4 or 16)
template <int A>
__device__ __forceinline__ void raw_load16(const uint8_t* p, uint32_t v[4])
{
  if constexpr (A >= 16) { const uint4 q = *reinterpret_cast<const uint4*>(p); v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w; }
  else if constexpr (A >= 4) {
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = reinterpret_cast<const uint32_t*>(p)[i];
  } else {
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = raw_u32_a2(p + 4 * i);
  }
}
__device__ __forceinline__ int raw_byte(const uint32_t v[4], int t) { return (int)((v[t >> 2] >> (8 * (t & 3))) & 0xffu); }

// Weights [16 * run, 16 * run + 16) of the row that starts at row_base.
template <int QT>
__device__ __forceinline__ void raw_run16(const uint8_t* row_base, int run, float w[16])
{
  constexpr int BB = raw_block_bytes(QT);
  if constexpr (QT == CAI_Q4_1 || QT == CAI_Q5_0 || QT == CAI_Q5_1) {
    const uint8_t* blk = row_base + (int64_t)(run >> 1) * BB;
    const int half = run & 1;
    uint32_t qs[4];
    raw_load16<QT == CAI_Q5_0 ? 2 : 4>(blk + (QT == CAI_Q4_1 ? 4 : QT == CAI_Q5_0 ? 6 : 8), qs);
    const float d = raw_half(blk);
    if constexpr (QT == CAI_Q4_1) {
      const float m = raw_half(blk + 2);
#pragma unroll
      for (int t = 0; t < 16; t++) { const int b = raw_byte(qs, t); w[t] = fmaf(d, (float)(half ? (b >> 4) : (b & 15)), m); }
    } else {
      const uint32_t qh = (QT == CAI_Q5_0 ? raw_u32_a2(blk + 2) : *reinterpret_cast<const uint32_t*>(blk + 4)) >> (16 * half);
      const float m = QT == CAI_Q5_1 ? raw_half(blk + 2) : 0.0f;
#pragma unroll
      for (int t = 0; t < 16; t++) {
        const int b = raw_byte(qs, t);
        const int q = (half ? (b >> 4) : (b & 15)) | (int)(((qh >> t) & 1u) << 4);
        w[t] = QT == CAI_Q5_0 ? d * (float)(q - 16) : fmaf(d, (float)q, m);
      }
    }
  } else {
    const uint8_t* blk = row_base + (int64_t)(run >> 4) * BB;
    const int r = run & 15;    // elements 16 r .. 16 r + 15 of the super-block
    if constexpr (QT == CAI_Q5_K) {
      const int c = r >> 2, hi = (r >> 1) & 1, half = r & 1, j = 2 * c + hi;
      int sc, mn; k_scale_min(blk + 4, j, sc, mn);
      const float dsc = raw_half(blk) * (float)sc, dm = raw_half(blk + 2) * (float)mn;
      uint32_t ql[4], qh[4];
      raw_load16<16>(blk + 48 + 32 * c + 16 * half, ql);
      raw_load16<16>(blk + 16 + 16 * half, qh);
#pragma unroll
      for (int t = 0; t < 16; t++) {
        const int b = raw_byte(ql, t);
        const int q = (hi ? (b >> 4) : (b & 15)) | (((raw_byte(qh, t) >> j) & 1) << 4);
        w[t] = fmaf(dsc, (float)q, -dm);
      }
    } else if constexpr (QT == CAI_Q2_K) {
      const uint8_t scb = blk[r];
      const float dl = raw_half(blk + 80) * (float)(scb & 15), ml = raw_half(blk + 82) * (float)(scb >> 4);
      uint32_t qs[4];
      raw_load16<4>(blk + 16 + (r >> 3) * 32 + 16 * (r & 1), qs);
      const int sh = 2 * ((r >> 1) & 3);
#pragma unroll
      for (int t = 0; t < 16; t++) w[t] = fmaf(dl, (float)((raw_byte(qs, t) >> sh) & 3), -ml);
    } else {   // Q3_K
      const float dl = raw_half(blk + 108) * (float)q3k_scale(blk + 96, r);
      uint32_t qs[4], hm[4];
      raw_load16<2>(blk + 32 + (r >> 3) * 32 + 16 * (r & 1), qs);
      raw_load16<2>(blk + 16 * (r & 1), hm);
      const int sh = 2 * ((r >> 1) & 3), bit = r >> 1;
#pragma unroll
      for (int t = 0; t < 16; t++) {
        const int clear = ((raw_byte(hm, t) >> bit) & 1) ^ 1;
        w[t] = dl * (float)(((raw_byte(qs, t) >> sh) & 3) - (clear << 2));
      }
    }
  }
}

}  // namespace cai
