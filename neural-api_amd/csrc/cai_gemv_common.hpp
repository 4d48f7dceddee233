// Device helpers and the launch-parameter block shared by the GEMV kernels (gfx950, wave64).
#pragma once
#include "cai_internal.hpp"

namespace cai {

// ------------------------------------------------------------------------------------------
// wave64 sum: DPP row_shr within rows of 16, then row_bcast15 / row_bcast31; total ends in lane 63.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v)
{
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, true)); // row_shr:1
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x112, 0xf, 0xf, true)); // row_shr:2
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, true)); // row_shr:4
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, true)); // row_shr:8
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, true)); // row_bcast:15
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, true)); // row_bcast:31
  return v;  // valid in lane 63
}

__device__ __forceinline__ float act_apply(float v, int act)
{
  // neural/neural.cl:114-146
  if (act == CAI_ACT_RELU) return v < 0.0f ? 0.0f : v;
  if (act == CAI_ACT_SIGMOID) {
    if (v > 0.0f) return 1.0f / (1.0f + expf(-v));
    const float s = expf(v); return s / (1.0f + s);
  }
  if (act == CAI_ACT_TANH) {
    float xc = v > 10.0f ? 10.0f : (v < -10.0f ? -10.0f : v);
    const float e = expf(-2.0f * xc); return (1.0f - e) / (1.0f + e);
  }
  return v;
}

__device__ __forceinline__ float silu_mul(float up, float gate)
{
  // neural/neural.cl:1236-1247: two-branch sigmoid, y = A * (B * sigmoid(B))
  float sig;
  if (gate > 0.0f) sig = 1.0f / (1.0f + expf(-gate));
  else { const float s = expf(gate); sig = s / (1.0f + s); }
  return up * (gate * sig);
}

constexpr int SSQ_PARTS = 1024;   // slots of a sum-of-squares partial array (>= any producer grid)

struct GemvSeg {
  const uint8_t* data; const uint8_t* aux; const float* bias;
  int rows;       // rows of this segment computed by the launch
  int y_off;      // offset of the segment's first output inside a y row
  int grp_end;    // cumulative row-group count (exclusive)
};

struct GemvParams {
  GemvSeg seg[3];
  int n_seg;
  const float* x;        // [NB][cols]
  float* y;              // [NB][y_stride]
  const float* residual; // same indexing as y, may be null
  const float* norm_gain; float norm_eps;  // fused RMSNorm on the input when norm_gain != null
  const float* ssq_in;   // optional: sum(x^2) as SSQ_PARTS partials written by the kernel that produced x
  float* ssq_out;        // optional: this kernel's per-work-group partials of sum(y^2) (SSQ_PARTS slots)
  int ssq_n;             // slots of the partial arrays in use (a multiple of 64, >= any producer grid on this device: the CU count rounded up)
  int cols;
  int kp;                // panel length in floats (multiple of 256)
  int kp_lds;            // LDS floats reserved per batch row: kp rounded up to whole 16-unit tiles
  int y_stride;
  int act;
  int half;              // swiglu: rows [0,half) are up, [half,2*half) gate
  // expert-bank gather (MoE): blockIdx.y = slot; the slot's expert id selects a row window of the bank
  const int32_t* slot_expert; int64_t expert_rows; int x_slot_stride; int y_slot_stride;
  int bank_experts;      // experts in the bank: a slot's id is clamped to [0, bank_experts) before it addresses rows
  // Q6_K: per segment the plane of d (kept behind the fields every launch reads: a wider segment record measured 2 % on the
  // launch-bound MoE step)
  const uint8_t* seg_aux2[3];
  unsigned long long* timeline;   // stamps of this launch's work-groups (null: none)
};

__device__ __forceinline__ float cvt_ub0(uint32_t v) { return (float)(v & 0xffu); }
__device__ __forceinline__ float cvt_ub1(uint32_t v) { return (float)((v >> 8) & 0xffu); }
__device__ __forceinline__ float cvt_ub2(uint32_t v) { return (float)((v >> 16) & 0xffu); }
__device__ __forceinline__ float cvt_ub3(uint32_t v) { return (float)(v >> 24); }

// Q4_K: the 6-bit (scale, min) pairs of sub-blocks 2cc and 2cc+1 from the 12 packed bytes
// (neural/neuralgguf.pas:448-464).  Returns packed bytes: sc = [sc_lo | sc_hi<<8], mn likewise.
__device__ __forceinline__ void q4k_scale_pair(uint32_t d0, uint32_t d1, uint32_t d2, int cc, uint32_t& sc, uint32_t& mn)
{
  const int sh = (cc & 1) * 16;
  const uint32_t h0 = (d0 >> sh) & 0xffffu, h1 = (d1 >> sh) & 0xffffu, h2 = (d2 >> sh) & 0xffffu;
  if (cc < 2) { sc = h0 & 0x3f3fu; mn = h1 & 0x3f3fu; }
  else { sc = (h2 & 0x0f0fu) | ((h0 >> 2) & 0x3030u); mn = ((h2 >> 4) & 0x0f0fu) | ((h1 >> 2) & 0x3030u); }
}


}  // namespace cai
