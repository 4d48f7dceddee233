/*
 * CPU ORACLE - TEST INFRASTRUCTURE, NOT PRODUCT CODE.  See oracle.h.
 *
 * Plain C restatement of the reference's quantized-decode arithmetic.
 * Pinning status of each function (what fixes it besides this text) is listed
 * in the comment above it; the tests under tests/ run those checks.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* scalar codecs                                                       */
/* ------------------------------------------------------------------ */

/* neural/neuralsafetensors.pas:294-329 (DecodeF16).
 * Pinned by: 21 known answers + Inf/NaN table of tests/TestNeuralVolume.pas:3223-3294,
 * and an exhaustive 65536-value sweep against the compiler's _Float16. */
float orc_f16_to_f32(uint16_t bits)
{
  uint32_t sign = (bits >> 15) & 1u, exponent = (bits >> 10) & 0x1Fu, mant = bits & 0x3FFu, o;
  float r;
  if (exponent == 0) {
    if (mant == 0) { o = sign << 31; memcpy(&r, &o, 4); return r; }
    r = (float)mant * 5.9604644775390625e-8f; /* m * 2^-24, exact */
    return sign ? -r : r;
  }
  if (exponent == 0x1F) o = (sign << 31) | (0xFFu << 23) | (mant << 13);
  else                  o = (sign << 31) | ((exponent + 112u) << 23) | (mant << 13);
  memcpy(&r, &o, 4);
  return r;
}

/* neural/neuralsafetensors.pas:338-396 (EncodeF16). Normal range rounds to nearest even;
 * the subnormal branch rounds on the single bit shifted out, as the reference does.
 * Pinned by: decode(encode(h)) == h for every finite half; normal range vs _Float16. */
uint16_t orc_f32_to_f16(float v)
{
  uint32_t bits, sign, ex, mant, half;
  int e;
  memcpy(&bits, &v, 4);
  sign = (bits >> 16) & 0x8000u; ex = (bits >> 23) & 0xFFu; mant = bits & 0x7FFFFFu;
  if (ex == 0xFF) return (uint16_t)(sign | (mant ? 0x7E00u : 0x7C00u));
  e = (int)ex - 127 + 15;
  if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u);
  if (e <= 0) {
    if (e < -10) return (uint16_t)sign;
    mant |= 0x800000u;
    half = mant >> (14 - e);
    if ((mant >> (13 - e)) & 1u) half++;
    return (uint16_t)(sign | half);
  }
  half = ((uint32_t)e << 10) | (mant >> 13);
  if (mant & 0x1000u) { if ((mant & 0xFFFu) || (half & 1u)) half++; }
  return (uint16_t)(sign | half);
}

/* neural/neuralgguf.pas:448-464 (DequantizeQ4KScaleMin == ggml get_scale_min_k4).
 * Pinned by: tiny_kquant golden vectors (through orc_dequant_q4_k) and a brute-force
 * check against the 6-bit field definition (tests build the 12 bytes from known sc/mn). */
void orc_q4k_scale_min(const uint8_t* p, uint8_t* sc, uint8_t* mn)
{
  for (int j = 0; j < 4; j++) {
    uint8_t d = p[j], m = p[j + 4], md = p[j + 8];
    sc[j]     = d & 0x3F;
    sc[j + 4] = (uint8_t)((md & 0x0F) | ((d >> 2) & 0x30));
    mn[j]     = m & 0x3F;
    mn[j + 4] = (uint8_t)((md >> 4) | ((m >> 2) & 0x30));
  }
}

/* ------------------------------------------------------------------ */
/* block geometry: neural/neuralgguf.pas:100-138                       */
/* ------------------------------------------------------------------ */
int64_t orc_block_elems(int type)
{
  switch (type) {
    case ORC_F32: case ORC_F16: case ORC_I8ROW: return 1;
    case ORC_Q4_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: case ORC_Q8_0: return 32;
    case ORC_Q2_K: case ORC_Q3_K: case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: return 256;
  }
  return -1;
}
int64_t orc_block_bytes(int type)
{
  switch (type) {
    case ORC_F32: return 4; case ORC_F16: return 2; case ORC_I8ROW: return 1;
    case ORC_Q4_0: return 18; case ORC_Q8_0: return 34; case ORC_Q4_K: return 144; case ORC_Q6_K: return 210;
    case ORC_Q4_1: return 20; case ORC_Q5_0: return 22; case ORC_Q5_1: return 24;    /* neuralgguf.pas:129-138 */
    case ORC_Q2_K: return 84; case ORC_Q3_K: return 110; case ORC_Q5_K: return 176;  /* neuralgguf.pas:115-125 */
  }
  return -1;
}
int64_t orc_row_bytes(int type, int64_t cols)
{
  int64_t be = orc_block_elems(type);
  if (be <= 0 || cols % be) return -1;
  return cols / be * orc_block_bytes(type);
}

/* ------------------------------------------------------------------ */
/* dequantizers                                                        */
/* ------------------------------------------------------------------ */

/* neural/neuralgguf.pas:1487-1503 -> TNNetVolume.DequantizeInt8 (neuralvolume.pas:12564-12582):
 * x = d * q, one single-precision multiply (exact: 11-bit x 7-bit significands).
 * Pinned by: closed form on hand-built blocks; tiny_llama_q8.gguf vs its fp32 twin. */
void orc_dequant_q8_0(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 34, out += 32) {
    uint16_t h; memcpy(&h, raw, 2);
    float d = orc_f16_to_f32(h);
    const int8_t* q = (const int8_t*)(raw + 2);
    for (int i = 0; i < 32; i++) out[i] = d * (float)q[i];
  }
}

/* neural/neuralgguf.pas:811-845 (LegacyNibble, DequantizeQ4_0): element e<16 is the low
 * nibble of byte e, e>=16 the high nibble of byte e-16; x = d * (nibble - 8).
 * Pinned by: the hand-built block of tests/TestNeuralPretrained.pas:6116-6143. */
void orc_dequant_q4_0(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 18, out += 32) {
    uint16_t h; memcpy(&h, raw, 2);
    float d = orc_f16_to_f32(h);
    const uint8_t* q = raw + 2;
    for (int e = 0; e < 32; e++) {
      int nib = (e < 16) ? (q[e] & 0x0F) : ((q[e - 16] >> 4) & 0x0F);
      out[e] = d * (float)(nib - 8);
    }
  }
}

/* neural/neuralgguf.pas:472-514 (DequantizeQ4K): x = (d*sc)*q - dmin*mn, evaluated as two
 * separate roundings-free products and one subtraction (see the exactness note in the
 * header of tests/test_oracle_dequant.py).
 * Pinned by: bit-exact against tests/fixtures/tiny_kquant_ref.json (1024 gguf-py values). */
void orc_dequant_q4_k(const uint8_t* raw, int64_t nb, float* out)
{
  uint8_t sc[8], mn[8];
  for (int64_t b = 0; b < nb; b++, raw += 144, out += 256) {
    uint16_t h0, h1; memcpy(&h0, raw, 2); memcpy(&h1, raw + 2, 2);
    float d = orc_f16_to_f32(h0), dmin = orc_f16_to_f32(h1);
    orc_q4k_scale_min(raw + 4, sc, mn);
    for (int c = 0; c < 4; c++) {
      volatile float dscLo = d * (float)sc[2 * c], dmLo = dmin * (float)mn[2 * c];
      volatile float dscHi = d * (float)sc[2 * c + 1], dmHi = dmin * (float)mn[2 * c + 1];
      const uint8_t* chunk = raw + 16 + 32 * c;
      float* lo = out + 64 * c; float* hi = lo + 32;
      for (int i = 0; i < 32; i++) {
        uint8_t pb = chunk[i];
        /* Exact result either way (the two products are exact and share a 2^-24 grid), so
         * fma contraction cannot change a bit; done in double to make that explicit. */
        lo[i] = (float)((double)dscLo * (double)(pb & 0x0F) - (double)dmLo);
        hi[i] = (float)((double)dscHi * (double)(pb >> 4) - (double)dmHi);
      }
    }
  }
}

/* neural/neuralgguf.pas:639-717 (DequantizeQ6K): 210-byte super-block = 128 B ql (low 4 bits), 64 B qh (high 2 bits),
 * 16 int8 group scales, f16 d.  Element i: ql byte (i/128)*64 + i%64, low nibble when i%128 < 64 else high; qh byte
 * (i/128)*32 + i%32, 2-bit field at shift 2*((i%128)/32); q = (ql | qh<<4) - 32; x = (d * scale[i/16]) * q.
 * d*scale has <= 18 significant bits and the product with q <= 24, so both roundings are exact. */
void orc_dequant_q6_k(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 210, out += 256) {
    const uint8_t* ql = raw; const uint8_t* qh = raw + 128; const int8_t* sc = (const int8_t*)(raw + 192);
    uint16_t h; memcpy(&h, raw + 208, 2);
    const float d = orc_f16_to_f32(h);
    for (int i = 0; i < 256; i++) {
      volatile float dl = d * (float)sc[i >> 4];
      const int lo = ql[(i >> 7) * 64 + (i & 63)];
      const int nib = (i & 127) < 64 ? (lo & 15) : (lo >> 4);
      const int hi2 = (qh[(i >> 7) * 32 + (i & 31)] >> (2 * ((i & 127) >> 5))) & 3;
      out[i] = dl * (float)((nib | (hi2 << 4)) - 32);
    }
  }
}

/* Packer for synthetic weights (the reference has none): per 16-group scale = max|x|/31 quantised to int8 against
 * d = max scale / 127, q = round(x / (d*scale)) clamped to [-32, 31]. */
void orc_quant_q6_k(const float* x, int64_t n, uint8_t* out)
{
  for (int64_t b = 0; b < n / 256; b++, x += 256, out += 210) {
    float gs[16], smax = 0.0f;
    for (int g = 0; g < 16; g++) {
      float a = 0.0f;
      for (int k = 0; k < 16; k++) { float v = fabsf(x[16 * g + k]); if (v > a) a = v; }
      gs[g] = a / 31.0f; if (gs[g] > smax) smax = gs[g];
    }
    const uint16_t dh = orc_f32_to_f16(smax / 127.0f);
    const float d = orc_f16_to_f32(dh);
    memset(out, 0, 210);
    memcpy(out + 208, &dh, 2);
    int8_t* sc = (int8_t*)(out + 192);
    for (int g = 0; g < 16; g++) {
      int s = d > 0.0f ? (int)lrintf(gs[g] / d) : 0;
      if (s > 127) s = 127;
      if (s < 1 && gs[g] > 0.0f) s = 1;
      sc[g] = (int8_t)s;
    }
    for (int i = 0; i < 256; i++) {
      const float dl = d * (float)sc[i >> 4];
      int q = dl > 0.0f ? (int)lrintf(x[i] / dl) : 0;
      if (q < -32) q = -32; if (q > 31) q = 31;
      const int u = q + 32;
      uint8_t* pl = out + (i >> 7) * 64 + (i & 63);
      if ((i & 127) < 64) *pl |= (uint8_t)(u & 15); else *pl |= (uint8_t)((u & 15) << 4);
      out[128 + (i >> 7) * 32 + (i & 31)] |= (uint8_t)((u >> 4) << (2 * ((i & 127) >> 5)));
    }
  }
}

/* neural/neuralgguf.pas:516-587 (DequantizeQ5K): 176-byte super-block = f16 d, f16 dmin, 12 packed scale bytes (the Q4_K
 * packing), 32 B qh (one bit plane: sub-block j takes bit j of byte i mod 32), 128 B ql (Q4_K's nibble layout);
 * q = ql | qh_bit << 4 in 0..31, x = (d*sc_j)*q - dmin*mn_j.  d*sc*q has <= 22 significant bits: every product is exact and
 * the subtraction rounds once, whatever the evaluation order.
 * Pinned by: bit-exact against tiny_kquant_ref.json["dequant"]["Q5_K"] (gguf-py values), tests/test_oracle_codecs.py. */
void orc_dequant_q5_k(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 176, out += 256) {
    uint16_t h; memcpy(&h, raw, 2); const float d = orc_f16_to_f32(h);
    memcpy(&h, raw + 2, 2); const float dmin = orc_f16_to_f32(h);
    uint8_t sc[8], mn[8]; orc_q4k_scale_min(raw + 4, sc, mn);
    const uint8_t* qh = raw + 16; const uint8_t* ql = raw + 48;
    for (int c = 0; c < 4; c++) {
      const int jlo = 2 * c;
      const float dsc_lo = d * (float)sc[jlo], dm_lo = dmin * (float)mn[jlo], dsc_hi = d * (float)sc[jlo + 1], dm_hi = dmin * (float)mn[jlo + 1];
      for (int i = 0; i < 32; i++) {
        const uint8_t qlb = ql[32 * c + i], qhb = qh[i];
        const int q_lo = (qlb & 0x0F) | (((qhb >> jlo) & 1) << 4), q_hi = (qlb >> 4) | (((qhb >> (jlo + 1)) & 1) << 4);
        out[64 * c + i] = (float)((double)dsc_lo * (double)q_lo - (double)dm_lo);
        out[64 * c + 32 + i] = (float)((double)dsc_hi * (double)q_hi - (double)dm_hi);
      }
    }
  }
}

/* neural/neuralgguf.pas:588-648 (DequantizeQ2K): 84-byte super-block = 16 bytes scale | min (low / high nibble, one per
 * 16-element sub-block), 64 B of 2-bit quants, f16 d, f16 dmin.  Element e: byte (e/128)*32 + e%32, field at shift
 * 2*((e%128)/32); x = (d*scale)*q - dmin*min.
 * Pinned by: bit-exact against tiny_kquant_ref.json["dequant"]["Q2_K"]. */
void orc_dequant_q2_k(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 84, out += 256) {
    uint16_t h; memcpy(&h, raw + 80, 2); const float d = orc_f16_to_f32(h);
    memcpy(&h, raw + 82, 2); const float dmin = orc_f16_to_f32(h);
    for (int e = 0; e < 256; e++) {
      const uint8_t scb = raw[e >> 4];
      const float dl = d * (float)(scb & 0x0F), ml = dmin * (float)(scb >> 4);
      const int q = (raw[16 + (e >> 7) * 32 + (e & 31)] >> (2 * ((e & 127) >> 5))) & 3;
      out[e] = (float)((double)dl * (double)q - (double)ml);
    }
  }
}

/* neural/neuralgguf.pas:718-806 (DequantizeQ3K): 110-byte super-block = 32 B hmask (third bit plane: bit e/32 of byte e%32),
 * 64 B qs (2-bit fields laid out like Q2_K), 12 bytes of 6-bit scales (bytes 0..7: low nibble = scale j, high = scale j+8;
 * bytes 8..11: two high bits of scales b, b+4, b+8, b+12 at shifts 0,2,4,6), f16 d.  scale = 6-bit value - 32;
 * q = ql - 4 when the hmask bit is CLEAR; x = (d*scale)*q.
 * Pinned by: the hand-built super-block of tests/TestNeuralPretrained.pas:6238-6299 (scales sb+24, codes e mod 4, hmask bit
 * (e mod 3) & 1) against its closed form; an independent vectorised restatement on random bytes. */
void orc_dequant_q3_k(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 110, out += 256) {
    const uint8_t* hm = raw; const uint8_t* qs = raw + 32; const uint8_t* sp = raw + 96;
    uint16_t h; memcpy(&h, raw + 108, 2); const float d = orc_f16_to_f32(h);
    for (int e = 0; e < 256; e++) {
      const int j = e >> 4;
      const int lsc = j < 8 ? (sp[j & 7] & 0x0F) : (sp[j & 7] >> 4);
      const int hsc = (sp[8 + (j & 3)] >> (2 * (j >> 2))) & 3;
      const float dl = d * (float)((lsc | (hsc << 4)) - 32);
      const int ql = (qs[(e >> 7) * 32 + (e & 31)] >> (2 * ((e & 127) >> 5))) & 3;
      const int qh = ((hm[e & 31] >> (e >> 5)) & 1) ^ 1;
      out[e] = dl * (float)(ql - (qh << 2));
    }
  }
}

/* Legacy 32-element blocks (neural/neuralgguf.pas:846-944); the nibble of element e is LegacyNibble (811-817): low nibble of
 * byte e for e < 16, high nibble of byte e - 16 otherwise; the fifth bit of Q5_x is bit e of a little-endian 32-bit plane.
 *   Q4_1 (20 B: f16 d, f16 m, 16 B nibbles):           x = d*nibble + m
 *   Q5_0 (22 B: f16 d, 4 B qh, 16 B nibbles):           x = d*((nibble | bit<<4) - 16)
 *   Q5_1 (24 B: f16 d, f16 m, 4 B qh, 16 B nibbles):    x = d*(nibble | bit<<4) + m
 * Pinned by: the hand-built blocks of tests/TestNeuralPretrained.pas:6145-6236 against their closed forms. */
static int legacy_nibble(const uint8_t* qs, int e) { return e < 16 ? (qs[e] & 0x0F) : (qs[e - 16] >> 4); }
void orc_dequant_q4_1(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 20, out += 32) {
    uint16_t h; memcpy(&h, raw, 2); const float d = orc_f16_to_f32(h);
    memcpy(&h, raw + 2, 2); const float m = orc_f16_to_f32(h);
    for (int e = 0; e < 32; e++) out[e] = (float)((double)d * (double)legacy_nibble(raw + 4, e) + (double)m);
  }
}
void orc_dequant_q5_0(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 22, out += 32) {
    uint16_t h; memcpy(&h, raw, 2); const float d = orc_f16_to_f32(h);
    uint32_t qh; memcpy(&qh, raw + 2, 4);
    for (int e = 0; e < 32; e++) out[e] = d * (float)((legacy_nibble(raw + 6, e) | (int)(((qh >> e) & 1u) << 4)) - 16);
  }
}
void orc_dequant_q5_1(const uint8_t* raw, int64_t nb, float* out)
{
  for (int64_t b = 0; b < nb; b++, raw += 24, out += 32) {
    uint16_t h; memcpy(&h, raw, 2); const float d = orc_f16_to_f32(h);
    memcpy(&h, raw + 2, 2); const float m = orc_f16_to_f32(h);
    uint32_t qh; memcpy(&qh, raw + 4, 4);
    for (int e = 0; e < 32; e++) out[e] = (float)((double)d * (double)(legacy_nibble(raw + 8, e) | (int)(((qh >> e) & 1u) << 4)) + (double)m);
  }
}

/* neural/neuralgguf.pas:1471-1523 (DecodeGGMLSpan) */
int orc_dequant(int type, const void* raw, int64_t n, float* out)
{
  const uint8_t* p = (const uint8_t*)raw;
  switch (type) {
    case ORC_F32: memcpy(out, raw, (size_t)n * 4); return 0;
    case ORC_F16: for (int64_t i = 0; i < n; i++) { uint16_t h; memcpy(&h, p + 2 * i, 2); out[i] = orc_f16_to_f32(h); } return 0;
    case ORC_Q8_0: if (n % 32) return -1; orc_dequant_q8_0(p, n / 32, out); return 0;
    case ORC_Q4_0: if (n % 32) return -1; orc_dequant_q4_0(p, n / 32, out); return 0;
    case ORC_Q4_K: if (n % 256) return -1; orc_dequant_q4_k(p, n / 256, out); return 0;
    case ORC_Q6_K: if (n % 256) return -1; orc_dequant_q6_k(p, n / 256, out); return 0;
    case ORC_Q5_K: if (n % 256) return -1; orc_dequant_q5_k(p, n / 256, out); return 0;
    case ORC_Q2_K: if (n % 256) return -1; orc_dequant_q2_k(p, n / 256, out); return 0;
    case ORC_Q3_K: if (n % 256) return -1; orc_dequant_q3_k(p, n / 256, out); return 0;
    case ORC_Q4_1: if (n % 32) return -1; orc_dequant_q4_1(p, n / 32, out); return 0;
    case ORC_Q5_0: if (n % 32) return -1; orc_dequant_q5_0(p, n / 32, out); return 0;
    case ORC_Q5_1: if (n % 32) return -1; orc_dequant_q5_1(p, n / 32, out); return 0;
  }
  return -2;
}

/* ------------------------------------------------------------------ */
/* quantizers                                                          */
/* ------------------------------------------------------------------ */

/* neural/neuralgguf.pas:1966-1989: d = amax/127, q = round-half-away(x/d) clamped to +-127.
 * Pinned by: |x - dequant(quant(x))| <= d/2 round trip; the reference writer's recipe. */
void orc_quant_q8_0(const float* x, int64_t n, uint8_t* out)
{
  for (int64_t b = 0; b < n / 32; b++, x += 32, out += 34) {
    float amax = 0;
    for (int i = 0; i < 32; i++) { float v = fabsf(x[i]); if (v > amax) amax = v; }
    float scale = amax / 127.0f, inv = scale == 0 ? 0 : 1.0f / scale;
    uint16_t h = orc_f32_to_f16(scale); memcpy(out, &h, 2);
    for (int i = 0; i < 32; i++) {
      float q = x[i] * inv;
      int e = q >= 0 ? (int)(q + 0.5f) : (int)(q - 0.5f);
      if (e > 127) e = 127; if (e < -127) e = -127;
      out[2 + i] = (uint8_t)(int8_t)e;
    }
  }
}

/* ggml quantize_row_q4_0_ref behaviour (not in the reference; this build's own definition):
 * d = (signed element of largest magnitude) / -8, q = min(15, (int)(x/d + 8.5)). */
void orc_quant_q4_0(const float* x, int64_t n, uint8_t* out)
{
  for (int64_t b = 0; b < n / 32; b++, x += 32, out += 18) {
    float amax = 0, mx = 0;
    for (int i = 0; i < 32; i++) { float v = fabsf(x[i]); if (v > amax) { amax = v; mx = x[i]; } }
    float d = mx / -8.0f, id = d == 0 ? 0 : 1.0f / d;
    uint16_t h = orc_f32_to_f16(d); memcpy(out, &h, 2);
    for (int e = 0; e < 16; e++) {
      int q0 = (int)(x[e] * id + 8.5f), q1 = (int)(x[e + 16] * id + 8.5f);
      if (q0 > 15) q0 = 15; if (q1 > 15) q1 = 15; if (q0 < 0) q0 = 0; if (q1 < 0) q1 = 0;
      out[2 + e] = (uint8_t)(q0 | (q1 << 4));
    }
  }
}

/* Simple affine Q4_K packer (this build's own; any valid packer is acceptable because the
 * dequantized values are the contract).  Per 32-sub-block: lo = min(0, min x), step =
 * (max-lo)/15; super-block d = max step / 63, dmin = max(-lo) / 63 (both stored as half);
 * sc = round(step/d), mn = round(-lo/dmin); q = round((x + dmin*mn)/(d*sc)) in 0..15.
 * Byte layout: neural/neuralgguf.pas:440-447 (6-bit packing) and 472-514 (nibbles). */
void orc_quant_q4_k(const float* x, int64_t n, uint8_t* out)
{
  for (int64_t b = 0; b < n / 256; b++, x += 256, out += 144) {
    float step[8], lo[8], maxstep = 0, maxneg = 0;
    for (int j = 0; j < 8; j++) {
      float mn_ = 0, mx_ = -INFINITY;
      for (int i = 0; i < 32; i++) { float v = x[32 * j + i]; if (v < mn_) mn_ = v; if (v > mx_) mx_ = v; }
      if (mx_ < mn_) mx_ = mn_;
      lo[j] = mn_; step[j] = (mx_ - mn_) / 15.0f;
      if (step[j] > maxstep) maxstep = step[j];
      if (-mn_ > maxneg) maxneg = -mn_;
    }
    uint16_t hd = orc_f32_to_f16(maxstep / 63.0f), hm = orc_f32_to_f16(maxneg / 63.0f);
    float d = orc_f16_to_f32(hd), dmin = orc_f16_to_f32(hm);
    uint8_t sc[8], mn[8];
    for (int j = 0; j < 8; j++) {
      int s = d > 0 ? (int)lrintf(step[j] / d) : 0, m = dmin > 0 ? (int)lrintf(-lo[j] / dmin) : 0;
      if (s > 63) s = 63; if (m > 63) m = 63; if (s < 0) s = 0; if (m < 0) m = 0;
      sc[j] = (uint8_t)s; mn[j] = (uint8_t)m;
    }
    memcpy(out, &hd, 2); memcpy(out + 2, &hm, 2);
    uint8_t* p = out + 4;
    for (int j = 0; j < 4; j++) {
      p[j]     = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
      p[j + 4] = (uint8_t)((mn[j] & 63) | ((mn[j + 4] >> 4) << 6));
      p[j + 8] = (uint8_t)((sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4));
    }
    for (int c = 0; c < 4; c++) {
      for (int i = 0; i < 32; i++) {
        int q[2];
        for (int hlf = 0; hlf < 2; hlf++) {
          int j = 2 * c + hlf;
          float ds = d * (float)sc[j], off = dmin * (float)mn[j];
          int v = ds > 0 ? (int)lrintf((x[32 * j + i] + off) / ds) : 0;
          if (v < 0) v = 0; if (v > 15) v = 15;
          q[hlf] = v;
        }
        out[16 + 32 * c + i] = (uint8_t)(q[0] | (q[1] << 4));
      }
    }
  }
}

/* neural/neuralvolume.pas:12501-12562 scalar twin: codes = round(v * (1/max) * 127) clamped
 * to +-127, scale = max/127 (callers: neural/neuralvolume.pas:926-987).  Round is
 * round-half-even (FPC Round / vcvtps2dq).  PARITY NOTE: the reference documents the tie
 * behaviour on boundary products as not bit-stable across its own builds
 * (neuralvolume.pas:728-735); pinned here by the round trip |x - scale*code| <= scale/2. */
void orc_quant_int8_row(const float* x, int64_t n, int8_t* codes, float* scale)
{
  float mx = 0;
  for (int64_t i = 0; i < n; i++) { float v = fabsf(x[i]); if (v > mx) mx = v; }
  *scale = mx / 127.0f;
  if (mx <= 0) { memset(codes, 0, (size_t)n); return; }
  float recip = 1.0f / mx;
  for (int64_t i = 0; i < n; i++) {
    float s = x[i] * recip * 127.0f;
    if (s > 127) s = 127; else if (s < -127) s = -127;
    codes[i] = (int8_t)lrintf(s);
  }
}

/* ------------------------------------------------------------------ */
/* row permutations                                                    */
/* ------------------------------------------------------------------ */

/* neural/neuralgguf.pas:428-438 */
int64_t orc_gguf_deinterleaved_src_row(int64_t hf_row, int head_dim)
{
  int64_t half = head_dim >> 1, r = hf_row % head_dim;
  if (r < half) return (hf_row - r) + 2 * r;
  return (hf_row - r) + 2 * (r - half) + 1;
}

/* neural/neuralpretrained.pas:14792-14812 (full-rotary case): HF row -> neuron index so that
 * interleaved-pair RoPE equals HF rotate_half. */
int64_t orc_map_target_neuron(int64_t row, int head_dim)
{
  int64_t half = head_dim >> 1, head = row / head_dim, r = row % head_dim;
  int64_t t = (r < half) ? 2 * r : 2 * (r - half) + 1;
  return head * head_dim + t;
}

/* ------------------------------------------------------------------ */
/* linear layer                                                        */
/* ------------------------------------------------------------------ */

/* neural.cl:114-146 activation tail (two-branch sigmoid, clamped tanh). */
static float apply_act(float v, int act)
{
  if (act == 1) return v < 0 ? 0 : v;
  if (act == 2) { if (v > 0) return 1.0f / (1.0f + expf(-v)); float s = expf(v); return s / (1.0f + s); }
  if (act == 3) { float xc = v > 10 ? 10 : (v < -10 ? -10 : v); float e = expf(-2.0f * xc); return (1.0f - e) / (1.0f + e); }
  return v;
}

/* Definition of the block-fused GEMV: dequantize the row exactly as the reference's loader
 * would (neuralgguf.pas:1471-1523), then Out[b*NumAs+a] = dot(W[a], X[b]) + bias[a]
 * (neuralvolume.pas:12127-12423 result layout; bias before activation, neural.cl:111-146).
 * ORC_I8ROW: scale applied once to the raw code sum (neuralvolume.pas:12693-12745).
 * Pinned by: definition (dequant is pinned above); fp32 vs double accumulation agree. */
int orc_gemv(int type, const void* raw, const float* scales, int64_t rows, int64_t cols,
             const float* x, int n_b, const float* bias, int act, int acc64, float* y)
{
  int64_t rb = orc_row_bytes(type, cols);
  if (rb < 0) return -1;
  int err = 0;
#pragma omp parallel
  {
    float* w = (float*)malloc((size_t)cols * sizeof(float));
#pragma omp for schedule(static)
    for (int64_t a = 0; a < rows; a++) {
      const uint8_t* rp = (const uint8_t*)raw + a * rb;
      if (type == ORC_I8ROW) { const int8_t* c = (const int8_t*)rp; for (int64_t i = 0; i < cols; i++) w[i] = (float)c[i]; }
      else if (orc_dequant(type, rp, cols, w)) { err = -2; continue; }
      for (int b = 0; b < n_b; b++) {
        const float* xb = x + (int64_t)b * cols;
        float r;
        if (acc64) { double s = 0; for (int64_t i = 0; i < cols; i++) s += (double)w[i] * (double)xb[i]; if (type == ORC_I8ROW) s *= (double)scales[a]; r = (float)s; }
        else       { float s = 0;  for (int64_t i = 0; i < cols; i++) s += w[i] * xb[i]; if (type == ORC_I8ROW) s *= scales[a]; r = s; }
        if (bias) r += bias[a];
        y[(int64_t)b * rows + a] = apply_act(r, act);
      }
    }
    free(w);
  }
  return err;
}

/* ------------------------------------------------------------------ */
/* elementwise layer math                                              */
/* ------------------------------------------------------------------ */

/* neural.cl:1047-1085 with FUseMean == 0: inv = 1/sqrt(mean(x^2)+eps); y = g*(x*inv). */
void orc_rmsnorm(const float* x, const float* gain, int n, float eps, float* y)
{
  float ss = 0;
  for (int c = 0; c < n; c++) ss = fmaf(x[c], x[c], ss);
  float inv = 1.0f / sqrtf(ss / (float)n + eps);
  for (int c = 0; c < n; c++) y[c] = gain[c] * (x[c] * inv);
}

/* Host-side frequency table the device kernel receives (neural.cl:1510-1515): theta_k =
 * base^(-2k/head_dim), computed in double and rounded once. */
void orc_rope_thetas(float base, int head_dim, float* th)
{
  for (int k = 0; k < head_dim / 2; k++) th[k] = (float)pow((double)base, -2.0 * k / head_dim);
}

/* Frequency table under a long-context rule (neural/neuralpretrained.pas:633-668: "linear" -> Position Interpolation,
 * "llama3" -> the Llama-3.1 rule with original_max_position_embeddings, low_freq_factor, high_freq_factor and NO output
 * scale; "dynamic"/"ntk" -> NTK-aware base change; "yarn" -> per-pair blend + attention temperature).  mode 0 none, 1 linear,
 * 2 llama3, 3 ntk, 4 yarn (low_freq_factor = beta_slow / YarnAlpha, high_freq_factor = beta_fast / YarnBeta, band edges
 * floored / ceiled as HF does by default).  The layer that applies the rule (TNNetRotaryEmbedding) is not among the
 * reference's files here, so the formulas are the published ones the importer's comments name: PI divides every frequency
 * by the factor; llama3 keeps pairs that turn more than high_freq_factor times over the original context, divides those
 * that turn less than low_freq_factor times, and blends linearly in the rotation count between.
 * Pinned by: the saturating case of tests/TestNeuralNumerical.pas:16008-16028 (d = 8, base 1e4, original 512, low 1,
 * high 4, factor 8: pairs 0, 1 kept, pairs 2, 3 divided by 8), theta/factor for linear, an independent float64 restatement
 * of the published rule on a 128-wide head (tests/test_oracle_model.py).  The llama3 blend region itself: parity unpinned
 * against the reference's layer (no fixture exercises it).  NTK: the exact formula of tests/TestNeuralNumerical.pas:15869-15880
 * (theta'_k = (base * s^(d/(d-2)))^(-2k/d)).  YaRN: the band case of tests/TestNeuralNumerical.pas:15890-15990 (d = 8, base 1e4,
 * original 512, s = 2, alpha 1, beta 32: low = floor(0.406) = 0, high = ceil(1.911) = 2, thetas 1, 0.075, 0.005, 0.0005 - the
 * blend of pair 1 included) and its temperature 0.1 ln(s) + 1 (orc_rope_out_scale). */
int orc_rope_thetas_scaled(float base, int head_dim, int mode, float factor, int original_ctx, float low_freq_factor, float high_freq_factor, float* th)
{
  if (mode < 0 || mode > 4 || !(factor >= 1.0f)) return -1;
  if ((mode == 2 || mode == 4) && (original_ctx <= 0 || !(high_freq_factor > low_freq_factor))) return -1;
  if (mode == 3 && head_dim <= 2) return -1;
  double ylow = 0.0, yhigh = 0.0;
  if (mode == 4) {   /* correction dims of beta_fast (high_freq_factor) and beta_slow (low_freq_factor) rotations */
    const double lb = 2.0 * log((double)base);
    ylow = floor(head_dim * log((double)original_ctx / ((double)high_freq_factor * 2.0 * M_PI)) / lb);
    yhigh = ceil(head_dim * log((double)original_ctx / ((double)low_freq_factor * 2.0 * M_PI)) / lb);
    if (ylow < 0.0) ylow = 0.0;
    if (yhigh > head_dim - 1) yhigh = head_dim - 1;
    if (yhigh == ylow) yhigh += 0.001;
  }
  for (int k = 0; k < head_dim / 2; k++) {
    const double t = pow((double)base, -2.0 * k / head_dim);
    double v = t;
    if (mode == 1) v = t / (double)factor;
    if (mode == 3) v = pow((double)base * pow((double)factor, (double)head_dim / (head_dim - 2.0)), -2.0 * k / head_dim);
    if (mode == 4) {
      double ramp = ((double)k - ylow) / (yhigh - ylow);
      ramp = ramp < 0.0 ? 0.0 : (ramp > 1.0 ? 1.0 : ramp);
      v = (t / (double)factor) * ramp + t * (1.0 - ramp);   /* ramp 0: keep the frequency; ramp 1: fully interpolated */
    }
    if (mode == 2) {
      const double wavelen = 2.0 * M_PI / t;
      const double lo_wl = (double)original_ctx / (double)low_freq_factor, hi_wl = (double)original_ctx / (double)high_freq_factor;
      if (wavelen < hi_wl) v = t;
      else if (wavelen > lo_wl) v = t / (double)factor;
      else {
        const double smooth = ((double)original_ctx / wavelen - (double)low_freq_factor) / ((double)high_freq_factor - (double)low_freq_factor);
        v = (1.0 - smooth) * t / (double)factor + smooth * t;
      }
    }
    th[k] = (float)v;
  }
  return 0;
}

/* The attention temperature a rule puts on the rotated q and k (the kernel's OutScale, neural.cl:1517-1542): YaRN
 * 0.1 ln(factor) + 1, every other rule 1. */
float orc_rope_out_scale(int mode, float factor) { return mode == 4 ? (float)(0.1 * log((double)factor) + 1.0) : 1.0f; }

/* neural.cl:1517-1542: pairs (2k,2k+1) per head, angle = (float)pos * theta_k (fp32 product). */
void orc_rope_interleaved(float* x, int n_heads, int head_dim, int pos, const float* th)
{
  for (int h = 0; h < n_heads; h++)
    for (int k = 0; k < head_dim / 2; k++) {
      float angle = (float)pos * th[k];
      float s = (float)sin((double)angle), c = (float)cos((double)angle);
      float* p = x + h * head_dim + 2 * k;
      float x0 = p[0], x1 = p[1];
      p[0] = c * x0 - s * x1;
      p[1] = s * x0 + c * x1;
    }
}

/* neural.cl:1213-1263 flag 1: y = A * (B * sigmoid(B)), A = first half (up), B = second (gate). */
void orc_swiglu(const float* ug, int half, float* y)
{
  for (int d = 0; d < half; d++) {
    float a = ug[d], b = ug[half + d], sig;
    if (b > 0) sig = 1.0f / (1.0f + expf(-b)); else { float s = expf(b); sig = s / (1.0f + s); }
    y[d] = a * (b * sig);
  }
}

/* neural.cl:1594-1647 with FApplyMinScale == 0 (TNNetPointwiseSoftMax). */
void orc_softmax(const float* x, int n, float* y)
{
  float mx = x[0];
  for (int c = 1; c < n; c++) if (x[c] > mx) mx = x[c];
  float tot = 0;
  for (int c = 0; c < n; c++) {
    float a = x[c] - mx; if (a > 4000) a = 4000; else if (a < -4000) a = -4000;
    y[c] = expf(a); tot += y[c];
  }
  if (tot > 0) { float inv = 1.0f / tot; for (int c = 0; c < n; c++) y[c] *= inv; }
}

/* TNNetTopKGate (source unavailable; known answer tests/TestNeuralNumerical.pas:74997-75042):
 * keep the k largest, zero the rest, optionally renormalise survivors to sum 1.  Ties: the
 * lower index is kept first (PARITY NOTE: tie rule not visible in the reference checkout).
 * idx_out lists survivors in descending value order. */
void orc_topk_gate(const float* p, int n, int k, int renorm, float* g, int* idx)
{
  char* used = (char*)calloc((size_t)n, 1);
  float sum = 0;
  for (int c = 0; c < n; c++) g[c] = 0;
  for (int j = 0; j < k; j++) {
    int best = -1;
    for (int c = 0; c < n; c++) if (!used[c] && (best < 0 || p[c] > p[best])) best = c;
    used[best] = 1; idx[j] = best; sum += p[best];
  }
  for (int j = 0; j < k; j++) g[idx[j]] = renorm ? (sum > 0 ? p[idx[j]] / sum : 0) : p[idx[j]];
  free(used);
}

/* neuralchatengine.pas:683-697 (ArgMaxRow): strict > from index 0, lowest index wins ties. */
int orc_argmax(const float* x, int n)
{
  int b = 0;
  for (int i = 1; i < n; i++) if (x[i] > x[b]) b = i;
  return b;
}

/* The distribution pipeline of TChatEngine.GenerateFromIds (neuralchatengine.pas:1374-1396, 1495-1501):
 * softmax of the logits row -> history penalty in the probability domain (neuralvolume.pas:5335-5376:
 * p^repetition, * exp(-(frequency*count + presence)) for every distinct token of the history, then / sum) ->
 * temperature in the probability domain (neuraldecode.pas:4710-4754: p := exp(ln(max(p,1e-30))/T - ln(max p)/T),
 * / sum, T clamped to >= 1e-6, T == 1 is a no-op) -> the candidate prefix the samplers draw from: the m most
 * probable tokens in descending order (TNNetSamplerBase.SelectTopCandidates + SortTokenArray, neuralvolume.pas:
 * 5171-5196; the reference's nucleus sampler starts from the same 256-wide prefix, 4548-4562).
 * Equal probabilities: lower token id first (the reference's quicksort leaves that order unspecified).
 * exp / ln / pow are libm's here; the reference uses its own polynomial versions (tolerance 1e-6, neural.cl:1660-1664).
 * Pinned by: softmax(logits / T) identity, closed-form penalty cases, sortedness and mass checks
 * (tests/test_oracle_sampling.py). */
typedef struct { float p; int32_t id; } orc_cand;
static int cand_cmp(const void* a, const void* b)
{
  const orc_cand* x = (const orc_cand*)a; const orc_cand* y = (const orc_cand*)b;
  if (x->p != y->p) return x->p > y->p ? -1 : 1;
  return x->id < y->id ? -1 : (x->id > y->id ? 1 : 0);
}

int orc_sample_candidates(const float* logits, int n, const int32_t* hist_ids, const int32_t* hist_counts, int n_hist,
                          float repetition, float frequency, float presence, float temperature, int m,
                          int32_t* tok_out, float* p_out)
{
  /* (row sums are accumulated in double: the reference's vectorised GetSum has its own order, and a sequential
   * float sum over a 152k row is off by ~1e-4 either way) */
  float* p = (float*)malloc((size_t)n * sizeof(float));
  {
    float mx = logits[0];
    for (int i = 1; i < n; i++) if (logits[i] > mx) mx = logits[i];
    double tot = 0;
    for (int i = 0; i < n; i++) {
      float a = logits[i] - mx; if (a > 4000) a = 4000; else if (a < -4000) a = -4000;
      p[i] = expf(a); tot += p[i];
    }
    if (tot > 0) { const float inv = (float)(1.0 / tot); for (int i = 0; i < n; i++) p[i] *= inv; }
  }
  if (repetition != 1.0f || frequency != 0.0f || presence != 0.0f) {
    int changed = 0;
    for (int k = 0; k < n_hist; k++) {
      const int t = hist_ids[k];
      if (t < 0 || t >= n) continue;
      float v = p[t];
      if (repetition != 1.0f && v > 0) v = powf(v, repetition);
      if (frequency != 0.0f || presence != 0.0f) v *= expf(-(frequency * (float)hist_counts[k] + presence));
      p[t] = v; changed = 1;
    }
    if (changed) {
      double tot = 0; for (int i = 0; i < n; i++) tot += p[i];
      if (tot > 0) for (int i = 0; i < n; i++) p[i] = (float)(p[i] / tot);
    }
  }
  if (temperature != 1.0f) {
    float T = temperature < 1e-6f ? 1e-6f : temperature;
    float mx = p[0]; for (int i = 1; i < n; i++) if (p[i] > mx) mx = p[i];
    if (mx > 0) {
      const float lm = logf(mx < 1e-30f ? 1e-30f : mx), inv_t = 1.0f / T;
      double sum = 0;
      for (int i = 0; i < n; i++) { float v = p[i] < 1e-30f ? 1e-30f : p[i]; v = expf(logf(v) * inv_t - lm * inv_t); p[i] = v; sum += v; }
      if (sum <= 0) sum = 1.0;
      const float inv = (float)(1.0 / sum);
      for (int i = 0; i < n; i++) p[i] *= inv;
    }
  }
  orc_cand* c = (orc_cand*)malloc((size_t)n * sizeof(orc_cand));
  for (int i = 0; i < n; i++) { c[i].p = p[i]; c[i].id = i; }
  qsort(c, (size_t)n, sizeof(orc_cand), cand_cmp);
  if (m > n) m = n;
  for (int i = 0; i < m; i++) { tok_out[i] = c[i].id; p_out[i] = c[i].p; }
  free(c); free(p);
  return m;
}

/* ------------------------------------------------------------------ */
/* attention                                                           */
/* ------------------------------------------------------------------ */

static float round_half(float v) { return orc_f16_to_f32(orc_f32_to_f16(v)); }

/* Live rows after `len` tokens: all of [j0, len) under a sliding window; under sink + recent-window eviction
 * (neuraldecode.pas:1257-1276: the first `sinks` positions and the latest `recent` are kept, the middle is gone, keys
 * keep their own rotation) positions [0, sinks) and [len - recent, len) once len exceeds sinks + recent.  The oracle
 * keeps every row and walks the live positions in order, so it states the policy, not a storage scheme.
 * Pinned by: within the cap identical to the unbounded run, row count pinned at the cap past it
 * (tests/TestNeuralDecode.pas:3863-3990), brute-force softmax over the stated set. */
static void live_runs(int len, int window, int sinks, int recent, int run0[2], int run1[2])
{
  /* at most two runs of consecutive positions, in ascending order */
  if (sinks + recent > 0 && len > sinks + recent) { run0[0] = 0; run1[0] = sinks; run0[1] = len - recent; run1[1] = len; }
  else { run0[0] = (window > 0 && len > window) ? len - window : 0; run1[0] = len; run0[1] = 0; run1[1] = 0; }
}

/* neural.cl:2354-2379 (append) + 2406-2499 (decode): scores q.K_j/sqrt(dk) (+softcap), max,
 * exp-shift, normaliser, out = (sum_j e_j V_j) * (1/sum).
 * Pinned by: tiny_*_logits.json through orc_model_step; brute-force softmax identity. */
static void attn_core_f32(const float* qkv, int hq, int hkv, int dk, float* kc, float* vc, int max_ctx,
                          int cache_len, int window, int sinks, int recent, float softcap, int kv_f16, float* out)
{
  const int qw = hq * dk, kw = hkv * dk, group = hq / hkv;
  for (int g = 0; g < hkv; g++)
    for (int d = 0; d < dk; d++) {
      float k = qkv[qw + g * dk + d], v = qkv[qw + kw + g * dk + d];
      if (kv_f16 == 1) { k = round_half(k); v = round_half(v); }
      kc[((int64_t)g * max_ctx + cache_len) * dk + d] = k;
      vc[((int64_t)g * max_ctx + cache_len) * dk + d] = v;
    }
  const int len = cache_len + 1;
  const float inv_sqrt = 1.0f / sqrtf((float)dk);
  float* sc = (float*)malloc((size_t)len * sizeof(float));
  /* the live rows are walked run by run, so a stream far past the cap costs what its live rows cost */
  int run0[2], run1[2];
  live_runs(len, window, sinks, recent, run0, run1);
  for (int h = 0; h < hq; h++) {
    const int g = h / group;
    const float* q = qkv + h * dk;
    float m = -1e30f;
    for (int r = 0; r < 2; r++)
      for (int j = run0[r]; j < run1[r]; j++) {
        const float* kr = kc + ((int64_t)g * max_ctx + j) * dk;
        float acc = 0;
        for (int d = 0; d < dk; d++) acc = fmaf(q[d], kr[d], acc);
        float s = acc * inv_sqrt;
        if (softcap > 0) s = softcap * tanhf(s / softcap);
        sc[j] = s; if (s > m) m = s;
      }
    float sum = 0;
    for (int r = 0; r < 2; r++)
      for (int j = run0[r]; j < run1[r]; j++) { sc[j] = expf(sc[j] - m); sum += sc[j]; }
    const float inv = sum > 0 ? 1.0f / sum : 0;
    for (int d = 0; d < dk; d++) {
      float acc = 0;
      for (int r = 0; r < 2; r++)
        for (int j = run0[r]; j < run1[r]; j++) acc = fmaf(sc[j], vc[((int64_t)g * max_ctx + j) * dk + d], acc);
      out[h * dk + d] = acc * inv;
    }
  }
  free(sc);
}

void orc_attn_decode(const float* qkv, int hq, int hkv, int dk, float* kc, float* vc, int max_ctx,
                     int cache_len, int window, float softcap, int kv_f16, float* out)
{
  attn_core_f32(qkv, hq, hkv, dk, kc, vc, max_ctx, cache_len, window, 0, 0, softcap, kv_f16, out);
}

void orc_attn_decode_evict(const float* qkv, int hq, int hkv, int dk, float* kc, float* vc, int max_ctx,
                           int cache_len, int sinks, int recent, float softcap, int kv_f16, float* out)
{
  attn_core_f32(qkv, hq, hkv, dk, kc, vc, max_ctx, cache_len, 0, sinks, recent, softcap, kv_f16, out);
}

/* neural.cl:2501-2580 (cai_sdpa_append_kv_int8), the device statement of the host's
 * QuantizeCacheRow: max over FINITE magnitudes (neuralvolume.pas:12471 MaxAbsFinite), a row whose
 * maximum is zero or denormal gets zero codes and unit scale, scale = max/127,
 * code = clamp(rint(v * (1/max) * 127)) with NaN -> 0 and +/-Inf -> +/-127.
 * Pinned by: the zero / one-outlier / flat / exact-midpoint rows of
 * tests/TestNeuralNumerical.pas:69740-69800 and the MaxAbsFinite cases of
 * tests/TestNeuralVolume.pas:2864-2903 (tests/test_oracle_kv_int8.py). */
float orc_max_abs_finite(const float* x, int n)
{
  float m = 0.0f;
  for (int i = 0; i < n; i++) {
    float a = fabsf(x[i]); uint32_t b; memcpy(&b, &a, 4);
    if (b <= 0x7F7FFFFFu && a > m) m = a;
  }
  return m;
}

void orc_kv_quant_row(const float* x, int n, int8_t* codes, float* scale)
{
  const float mx = orc_max_abs_finite(x, n);
  uint32_t mb; memcpy(&mb, &mx, 4);
  const int usable = mb >= 0x00800000u;
  const float recip = usable ? 1.0f / mx : 0.0f;
  *scale = usable ? mx / 127.0f : 1.0f;
  for (int i = 0; i < n; i++) {
    float a = fabsf(x[i]); uint32_t b; memcpy(&b, &a, 4);
    float scaled = x[i] * recip * 127.0f;
    if (b > 0x7F800000u || !usable) scaled = 0.0f;   /* an unusable row is all zero codes (neuralvolume.pas:725) */
    float r = rintf(scaled);                 /* half-to-even under the default rounding mode */
    if (r < -127.0f) r = -127.0f;
    if (r > 127.0f) r = 127.0f;
    codes[i] = (int8_t)r;
  }
}

/* neural.cl:2582-2687 (cai_sdpa_decode_int8): same phases as the fp32 kernel; the K row scale
 * multiplies the finished dot product together with 1/sqrt(dk), the V row scale multiplies the
 * softmax weight, the codes enter the accumulators as integers-in-float.
 * Pinned by: agreement with orc_attn_decode on caches whose rows quantise exactly
 * (tests/test_oracle_kv_int8.py), plus orc_kv_quant_row's vectors for the append. */
void orc_attn_decode_i8(const float* qkv, int hq, int hkv, int dk, int8_t* kq, float* ks, int8_t* vq, float* vs,
                        int max_ctx, int cache_len, int window, float softcap, float* out)
{
  const int qw = hq * dk, kw = hkv * dk, group = hq / hkv;
  for (int g = 0; g < hkv; g++) {
    const int64_t slot = (int64_t)g * max_ctx + cache_len;
    orc_kv_quant_row(qkv + qw + g * dk, dk, kq + slot * dk, ks + slot);
    orc_kv_quant_row(qkv + qw + kw + g * dk, dk, vq + slot * dk, vs + slot);
  }
  const int len = cache_len + 1;
  const int j0 = (window > 0 && len > window) ? len - window : 0;
  const float inv_sqrt = 1.0f / sqrtf((float)dk);
  float* sc = (float*)malloc((size_t)len * sizeof(float));
  for (int h = 0; h < hq; h++) {
    const int g = h / group;
    const float* q = qkv + h * dk;
    float m = -1e30f;
    for (int j = j0; j < len; j++) {
      const int8_t* kr = kq + ((int64_t)g * max_ctx + j) * dk;
      float acc = 0;
      for (int d = 0; d < dk; d++) acc = fmaf(q[d], (float)kr[d], acc);
      float s = acc * (ks[(int64_t)g * max_ctx + j] * inv_sqrt);
      if (softcap > 0) s = softcap * tanhf(s / softcap);
      sc[j] = s; if (s > m) m = s;
    }
    float sum = 0;
    for (int j = j0; j < len; j++) { sc[j] = expf(sc[j] - m); sum += sc[j]; }
    const float inv = sum > 0 ? 1.0f / sum : 0;
    for (int d = 0; d < dk; d++) {
      float acc = 0;
      for (int j = j0; j < len; j++)
        acc = fmaf(sc[j] * vs[(int64_t)g * max_ctx + j], (float)vq[((int64_t)g * max_ctx + j) * dk + d], acc);
      out[h * dk + d] = acc * inv;
    }
  }
  free(sc);
}

/* ------------------------------------------------------------------ */
/* whole decoder                                                       */
/* ------------------------------------------------------------------ */

typedef struct { int type; int64_t rows, cols; const void* raw; const float* scales; const float* bias; } orc_tensor;

typedef struct {
  orc_tensor w[9];
  const float* v[5];
  float *kc, *vc;
  int8_t *kq, *vq; float *ks, *vs;   /* int8 cache mode */
} orc_layer;

struct orc_model {
  orc_config cfg;
  orc_tensor embed, head;
  const float* final_norm;
  orc_layer* layers;
  float* theta;
  float rope_out_scale;   /* multiplies the rotated q and k (1 unless a rule sets it) */
  int len;
  float *x, *h, *qkv, *att, *gu, *mid, *tmp, *probs, *gates, *logits;
  float *probs_all;   /* router probabilities of every block at the last step (a test's view of how close a selection was) */
  int swap_layer, swap_pos;   /* test hook: at this block and position the k-th and (k+1)-th expert trade places (-1: never) */
  int* sel;
};

orc_model* orc_model_new(const orc_config* cfg)
{
  orc_model* m = (orc_model*)calloc(1, sizeof(*m));
  m->cfg = *cfg;
  const int L = cfg->n_layers, d = cfg->d_model, qw = cfg->n_q_heads * cfg->head_dim, kw = cfg->n_kv_heads * cfg->head_dim;
  m->layers = (orc_layer*)calloc((size_t)L, sizeof(orc_layer));
  for (int l = 0; l < L; l++) {
    m->layers[l].kc = (float*)calloc((size_t)kw * cfg->max_ctx, sizeof(float));
    m->layers[l].vc = (float*)calloc((size_t)kw * cfg->max_ctx, sizeof(float));
    if (cfg->kv_f16 == 2) {
      m->layers[l].kq = (int8_t*)calloc((size_t)kw * cfg->max_ctx, 1); m->layers[l].vq = (int8_t*)calloc((size_t)kw * cfg->max_ctx, 1);
      m->layers[l].ks = (float*)calloc((size_t)cfg->n_kv_heads * cfg->max_ctx, 4); m->layers[l].vs = (float*)calloc((size_t)cfg->n_kv_heads * cfg->max_ctx, 4);
    }
  }
  m->theta = (float*)malloc(sizeof(float) * (size_t)(cfg->head_dim / 2));
  orc_rope_thetas(cfg->rope_theta, cfg->head_dim, m->theta);
  m->rope_out_scale = 1.0f;
  int wide = d; if (qw > wide) wide = qw;
  m->x = (float*)calloc((size_t)d, 4); m->h = (float*)calloc((size_t)wide, 4);
  m->qkv = (float*)calloc((size_t)(qw + 2 * kw), 4); m->att = (float*)calloc((size_t)qw, 4);
  m->gu = (float*)calloc((size_t)2 * cfg->ffn, 4); m->mid = (float*)calloc((size_t)cfg->ffn, 4);
  m->tmp = (float*)calloc((size_t)wide, 4);
  int ne = cfg->n_experts > 0 ? cfg->n_experts : 1;
  m->swap_layer = -1; m->swap_pos = -1;
  m->probs_all = (float*)calloc((size_t)ne * (size_t)(cfg->n_layers > 0 ? cfg->n_layers : 1), 4);
  m->probs = (float*)calloc((size_t)ne, 4); m->gates = (float*)calloc((size_t)ne, 4); m->sel = (int*)calloc((size_t)ne, sizeof(int));
  m->logits = (float*)calloc((size_t)cfg->vocab, 4);
  return m;
}

void orc_model_free(orc_model* m)
{
  if (!m) return;
  for (int l = 0; l < m->cfg.n_layers; l++) { orc_layer* y = &m->layers[l]; free(y->kc); free(y->vc); free(y->kq); free(y->vq); free(y->ks); free(y->vs); }
  free(m->layers); free(m->theta); free(m->x); free(m->h); free(m->qkv); free(m->att); free(m->gu); free(m->mid);
  free(m->probs_all);
  free(m->tmp); free(m->probs); free(m->gates); free(m->sel); free(m->logits); free(m);
}

int orc_model_set_tensor(orc_model* m, int layer, int slot, int type, int64_t rows, int64_t cols,
                         const void* raw, const float* scales, const float* bias)
{
  orc_tensor t = { type, rows, cols, raw, scales, bias };
  if (slot == ORC_W_EMBED) { m->embed = t; return 0; }
  if (slot == ORC_W_HEAD) { m->head = t; return 0; }
  if (layer < 0 || layer >= m->cfg.n_layers || slot < 2 || slot > 8) return -1;
  m->layers[layer].w[slot] = t;
  return 0;
}

int orc_model_set_vec(orc_model* m, int layer, int slot, const float* v, int n)
{
  (void)n;
  if (slot == ORC_V_FINAL_NORM) { m->final_norm = v; return 0; }
  if (layer < 0 || layer >= m->cfg.n_layers || slot < 0 || slot > 4) return -1;
  m->layers[layer].v[slot] = v;
  return 0;
}

/* replaces the model's frequency table (head_dim / 2 values): long-context rules only change the table */
void orc_model_set_thetas(orc_model* m, const float* th, int n)
{
  if (n == m->cfg.head_dim / 2) memcpy(m->theta, th, sizeof(float) * (size_t)n);
}

void orc_model_set_rope_out_scale(orc_model* m, float s) { m->rope_out_scale = s; }

void orc_model_reset(orc_model* m) { m->len = 0; }
void orc_model_truncate(orc_model* m, int n) { if (n < m->len) m->len = n < 0 ? 0 : n; }
int  orc_model_len(const orc_model* m) { return m->len; }

static void lin(const orc_model* m, const orc_tensor* t, int64_t row0, int64_t rows, const float* x, float* y)
{
  int64_t rb = orc_row_bytes(t->type, t->cols);
  orc_gemv(t->type, (const uint8_t*)t->raw + row0 * rb, t->scales ? t->scales + row0 : 0, rows, t->cols, x, 1,
           t->bias ? t->bias + row0 : 0, 0, m->cfg.acc64, y);
}

/* One decode step in the reference's graph order (neuralpretrained.pas:16384-16882 builds it;
 * neuraldecode.pas:5696-5712 StepForward runs it): embedding row -> per block { RMSNorm ->
 * q,k,v (+bias) -> [full-width q/k RMSNorm] -> interleaved RoPE -> cached GQA -> o -> +res ->
 * RMSNorm -> gate|up -> SwiGLU -> down -> +res } -> final RMSNorm -> head -> argmax.
 * MoE FFN (neuralpretrained.pas:15331-15388): router -> softmax over all experts -> top-k
 * (renorm iff norm_topk) -> sum_e g_e * down_e(SwiGLU(gateup_e(h))).
 * Pinned by: tests/fixtures/tiny_{llama,smollm2,qwen2,mistral,olmoe}_logits.json (< 1e-4). */
int orc_model_step(orc_model* m, int token, int pos, float* logits)
{
  const orc_config* c = &m->cfg;
  const int d = c->d_model, hd = c->head_dim, qw = c->n_q_heads * hd, kw = c->n_kv_heads * hd, I = c->ffn;
  if (pos != m->len || pos >= c->max_ctx || token < 0 || token >= c->vocab) return -1;
  {
    int64_t rb = orc_row_bytes(m->embed.type, m->embed.cols);
    if (m->embed.type == ORC_I8ROW) {
      const int8_t* cd = (const int8_t*)m->embed.raw + (int64_t)token * rb;
      for (int i = 0; i < d; i++) m->x[i] = (float)cd[i] * m->embed.scales[token]; /* neural.cl:1447-1470 */
    } else orc_dequant(m->embed.type, (const uint8_t*)m->embed.raw + (int64_t)token * rb, d, m->x);
  }
  for (int l = 0; l < c->n_layers; l++) {
    orc_layer* ly = &m->layers[l];
    orc_rmsnorm(m->x, ly->v[ORC_V_ATTN_NORM], d, c->eps, m->h);
    lin(m, &ly->w[ORC_W_Q], 0, qw, m->h, m->qkv);
    lin(m, &ly->w[ORC_W_K], 0, kw, m->h, m->qkv + qw);
    lin(m, &ly->w[ORC_W_V], 0, kw, m->h, m->qkv + qw + kw);
    if (c->qk_norm_full) {
      orc_rmsnorm(m->qkv, ly->v[ORC_V_Q_NORM], qw, c->eps, m->tmp); memcpy(m->qkv, m->tmp, (size_t)qw * 4);
      orc_rmsnorm(m->qkv + qw, ly->v[ORC_V_K_NORM], kw, c->eps, m->tmp); memcpy(m->qkv + qw, m->tmp, (size_t)kw * 4);
    }
    orc_rope_interleaved(m->qkv, c->n_q_heads, hd, pos, m->theta);
    orc_rope_interleaved(m->qkv + qw, c->n_kv_heads, hd, pos, m->theta);
    if (m->rope_out_scale != 1.0f) for (int i = 0; i < qw + kw; i++) m->qkv[i] *= m->rope_out_scale;
    if (c->kv_f16 == 2) orc_attn_decode_i8(m->qkv, c->n_q_heads, c->n_kv_heads, hd, ly->kq, ly->ks, ly->vq, ly->vs, c->max_ctx, pos, c->window, 0.0f, m->att);
    else attn_core_f32(m->qkv, c->n_q_heads, c->n_kv_heads, hd, ly->kc, ly->vc, c->max_ctx, pos, c->window, c->evict_sinks, c->evict_recent, 0.0f, c->kv_f16, m->att);
    lin(m, &ly->w[ORC_W_O], 0, d, m->att, m->tmp);
    for (int i = 0; i < d; i++) m->x[i] += m->tmp[i];
    orc_rmsnorm(m->x, ly->v[ORC_V_MLP_NORM], d, c->eps, m->h);
    if (c->n_experts > 0) {
      lin(m, &ly->w[ORC_W_ROUTER], 0, c->n_experts, m->h, m->tmp);
      orc_softmax(m->tmp, c->n_experts, m->probs);
      memcpy(m->probs_all + (size_t)l * c->n_experts, m->probs, (size_t)c->n_experts * 4);
      if (l == m->swap_layer && pos == m->swap_pos && c->top_k < c->n_experts) {
        /* the selection a rounding-level change of the router sums would make: rank top_k and rank top_k + 1 trade their
         * probabilities (ranks by value, lower index first on equal values, as orc_topk_gate orders them) */
        int ik = -1, ik1 = -1;
        for (int i = 0; i < c->n_experts; i++) {
          int rank = 0;
          for (int j = 0; j < c->n_experts; j++) if (m->probs[j] > m->probs[i] || (m->probs[j] == m->probs[i] && j < i)) rank++;
          if (rank == c->top_k - 1) ik = i;
          if (rank == c->top_k) ik1 = i;
        }
        if (ik >= 0 && ik1 >= 0) { float t = m->probs[ik]; m->probs[ik] = m->probs[ik1]; m->probs[ik1] = t; }
      }
      orc_topk_gate(m->probs, c->n_experts, c->top_k, c->norm_topk, m->gates, m->sel);
      float* acc = (float*)calloc((size_t)d, 4);
      for (int j = 0; j < c->top_k; j++) {
        int e = m->sel[j];
        lin(m, &ly->w[ORC_W_GATEUP], (int64_t)e * 2 * I, 2 * I, m->h, m->gu);
        orc_swiglu(m->gu, I, m->mid);
        lin(m, &ly->w[ORC_W_DOWN], (int64_t)e * d, d, m->mid, m->tmp);
        for (int i = 0; i < d; i++) acc[i] = fmaf(m->gates[e], m->tmp[i], acc[i]); /* neural.cl:2738-2748 */
      }
      for (int i = 0; i < d; i++) m->x[i] += acc[i];
      free(acc);
    } else {
      lin(m, &ly->w[ORC_W_GATEUP], 0, 2 * I, m->h, m->gu);
      orc_swiglu(m->gu, I, m->mid);
      lin(m, &ly->w[ORC_W_DOWN], 0, d, m->mid, m->tmp);
      for (int i = 0; i < d; i++) m->x[i] += m->tmp[i];
    }
  }
  orc_rmsnorm(m->x, m->final_norm, d, c->eps, m->h);
  const orc_tensor* hw = m->head.raw ? &m->head : &m->embed; /* tied head: neuralpretrained.pas:15555- */
  lin(m, hw, 0, c->vocab, m->h, m->logits);
  if (logits) memcpy(logits, m->logits, (size_t)c->vocab * 4);
  m->len = pos + 1;
  return orc_argmax(m->logits, c->vocab);
}

/* HiddenState (neural/neuraldecode.pas:5850-5857): the output of the layer feeding the vocabulary projection, which in the
 * imported decoders is the final TokenRMSNorm (neuralpretrained.pas:16872-16875).  The step above keeps it in m->h. */
const float* orc_model_hidden(const orc_model* m) { return m->h; }
/* test hook: the step at position `pos` selects, in block `layer`, the (k+1)-th most probable expert instead of the k-th
 * (what the other side of a near tie looks like); layer -1 switches it off */
void orc_model_swap_selection(orc_model* m, int layer, int pos) { m->swap_layer = layer; m->swap_pos = pos; }
/* router probabilities (soft-max over all experts) of block `layer` at the last step; null for a dense model */
const float* orc_model_router_probs(const orc_model* m, int layer)
{
  if (m->cfg.n_experts <= 0 || layer < 0 || layer >= m->cfg.n_layers) return 0;
  return m->probs_all + (size_t)layer * m->cfg.n_experts;
}

/* ------------------------------------------------------------------------------------------
 * Prompt-lookup draft (neural/neuraldecode.pas:7742-7765), kept in the reference's own 1-based terms: the suffix is
 * Context[CtxLen-MatchLen+1 .. CtxLen]; candidate starts P run from CtxLen-MatchLen down to 1 (P = CtxLen-MatchLen+1 would be
 * the suffix itself); at the first P whose MatchLen tokens equal the suffix, FollowLen = CtxLen-(P+MatchLen)+1 tokens are
 * available after the match, of which at most NumDraft are copied; the scan stops there whether or not anything was copied.
 * Pinned by hand-derived cases and by an exhaustive comparison with the definition restated over all start positions on
 * short contexts of a two- and three-letter alphabet (tests/test_oracle_lookup.py).
 * ------------------------------------------------------------------------------------------ */
int orc_prompt_lookup_draft(const int32_t* ctx, int n_ctx, int match_len, int num_draft, int32_t* draft)
{
  const int CtxLen = n_ctx;
  if (match_len < 1 || num_draft < 1 || CtxLen < match_len + 1) return 0;
  const int SuffixStart = CtxLen - match_len + 1;             /* 1-based */
  for (int P = CtxLen - match_len; P >= 1; P--) {
    int equal = 1;
    for (int i = 0; i < match_len; i++)
      if (ctx[P - 1 + i] != ctx[SuffixStart - 1 + i]) { equal = 0; break; }
    if (!equal) continue;
    int FollowLen = CtxLen - (P + match_len) + 1;
    if (FollowLen > num_draft) FollowLen = num_draft;
    if (FollowLen < 1) return 0;
    for (int i = 0; i < FollowLen; i++) draft[i] = ctx[P + match_len - 1 + i];
    return FollowLen;
  }
  return 0;
}
