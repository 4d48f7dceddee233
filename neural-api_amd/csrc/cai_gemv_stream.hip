// Persistent streaming Q4_K matrix-vector kernel for batch-1 decode on gfx950.
//
// A fixed number of work-groups (a few per CU) stays resident and strides over the matrix's row groups.
// One lane owns one pair of Q4_K sub-blocks (64 weights = two 128-bit loads of quants + the 16-byte
// super-block header); a wave covers 16 super-blocks (4096 columns).  Rows longer than that are split over
// `nsw` waves of the work-group, each owning a fixed column slice, so every wave keeps ITS slice of the
// activation vector in registers for the whole kernel (loaded once, token RMSNorm fused into that load) and
// the inner loop touches neither LDS nor the activation again.  Weights for the next row group are
// requested before the current group is reduced (two register slots, no copies), so the HBM pipe stays full.
// Row sums: DPP reduction inside the wave, then (nsw > 1) a tiny LDS exchange between the slice waves.
//
// Semantics: Out[a] = act(dot(W[a], X) + bias[a]) (+ residual), or for the fused feed-forward front half
// Out[i] = up_i * silu(gate_i) with up = row i and gate = row half + i
// (reference: neural/neuralvolume.pas:12127-12423; neural/neural.cl:111-146, 1047-1085, 1213-1263).
#include "cai_gemv_common.hpp"

namespace cai {

struct Q4kRegs { uint4 h, q0, q1; };

// LDS slot (in float4) of the t-th float4 (t = 0..15) of unit u (= sb*4 + cc): tiles of 16 units, transposed
__device__ __forceinline__ int xs_slot(int u, int t) { return (u >> 4) * 256 + t * 16 + (u & 15); }

template <int R, int MODE, bool MULTISEG>
__global__ __launch_bounds__(512, (MODE == 1 ? 2 * R : R) <= 2 ? 3 : 2) void gemv_q4k_stream(const GemvParams p, const int n_groups, const int nsw, const int gwv)
{
  extern __shared__ float4 xs4[];
  constexpr int RR = MODE == 1 ? 2 * R : R;
  __shared__ float s_ss[16];
  constexpr int CH = 4;                       // row groups between two meetings of the slice waves
  __shared__ float s_part[2][8][CH][RR];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int step = wave % nsw, gslot = wave / nsw;
  const int cols = p.cols, nsb = cols >> 8;
  const int64_t row_bytes = (int64_t)nsb * 144;
  const int sb = step * 16 + (lane >> 2), cc = lane & 3;
  const bool act = sb < nsb;
  const int g_first = blockIdx.x * gwv + gslot, g_stride = gridDim.x * gwv;
  const int n_iters = (n_groups + g_stride - 1) / g_stride;
  const int64_t lane_off = (int64_t)(act ? sb : 0) * 144;

  // group -> segment, first row of the group inside the segment
  auto locate = [&](int g, const GemvSeg*& sg, int& row0) {
    int s = 0, g0 = 0;
    if (MULTISEG) {
      if (p.n_seg > 1 && g >= p.seg[0].grp_end) { s = 1; g0 = p.seg[0].grp_end; }
      if (p.n_seg > 2 && g >= p.seg[1].grp_end) { s = 2; g0 = p.seg[1].grp_end; }
    }
    sg = &p.seg[s]; row0 = (g - g0) * R;
  };
  auto issue = [&](int g, Q4kRegs (&rg)[RR]) {
    if (g < n_groups && act) {
      const GemvSeg* sg; int row0; locate(g, sg, row0);
      const int lim = MODE == 1 ? p.half : sg->rows;
#pragma unroll
      for (int r = 0; r < RR; r++) {
        int row = row0 + (MODE == 1 ? (r >> 1) : r);
        if (row >= lim) row = lim - 1;               // tail group: re-read the last row, result is not written
        if (MODE == 1 && (r & 1)) row += p.half;
        const uint8_t* blk = sg->data + (int64_t)row * row_bytes + lane_off;
        rg[r].h = *reinterpret_cast<const uint4*>(blk);
        rg[r].q0 = *reinterpret_cast<const uint4*>(blk + 16 + 32 * cc);
        rg[r].q1 = *reinterpret_cast<const uint4*>(blk + 32 + 32 * cc);
      }
    }
  };

  Q4kRegs buf0[RR], buf1[RR];
  issue(g_first, buf0);   // weights do not depend on the activation: request them before anything else

  float xv[64];
#pragma unroll
  for (int i = 0; i < 64; i++) xv[i] = 0.0f;
  bool staged;
  // ---- activation: staged once per work-group into LDS (unit-transposed tiles: 16 adjacent lanes read 16 adjacent
  //      float4), RMSNorm fused into the staging pass; then every wave lifts ITS 64 values into registers ----
  {
    float inv = 1.0f;
    if (p.norm_gain && p.ssq_in) {
      // sum of squares of x delivered by the producing kernel as SSQ_PARTS per-work-group partials (fixed order)
      float t = 0.0f;
#pragma unroll
      for (int i = 0; i < SSQ_PARTS / 64; i++) t += p.ssq_in[i * 64 + lane];
      t = wave_sum(t);
      t = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, t), 63));
      inv = 1.0f / sqrtf(t / (float)cols + p.norm_eps);
    }
    const float4* src = reinterpret_cast<const float4*>(p.x);
    const float4* gsrc = reinterpret_cast<const float4*>(p.norm_gain);
    const int n4 = cols >> 2, nthr = blockDim.x;
    float ss = 0.0f;
    const bool direct = gwv == 1 && !(p.norm_gain && !p.ssq_in);   // disjoint slices: LDS would only add a barrier
    if (direct) {
      if (act) {
        const int n0 = (sb * 4 + cc) * 16;
#pragma unroll
        for (int t = 0; t < 16; t++) {
          float4 v = src[n0 + t];
          if (p.norm_gain) {
            const float4 g = gsrc[n0 + t];
            v.x = g.x * (v.x * inv); v.y = g.y * (v.y * inv); v.z = g.z * (v.z * inv); v.w = g.w * (v.w * inv);
          }
          xv[4 * t] = v.x; xv[4 * t + 1] = v.y; xv[4 * t + 2] = v.z; xv[4 * t + 3] = v.w;
        }
      }
    } else
    for (int n = threadIdx.x; n < n4; n += nthr) {
      float4 v = src[n];
      if (p.norm_gain) {
        if (p.ssq_in) {
          const float4 g = gsrc[n];
          v.x = g.x * (v.x * inv); v.y = g.y * (v.y * inv); v.z = g.z * (v.z * inv); v.w = g.w * (v.w * inv);
        } else { ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss); }
      }
      xs4[xs_slot(n >> 4, n & 15)] = v;     // n = [sb][cc:2][t:4] -> unit sb*4+cc, float4 t
    }
    if (p.norm_gain && !p.ssq_in) {          // stand-alone call: reduce here, then rescale the entries this thread wrote
      ss = wave_sum(ss);
      if (lane == 63) s_ss[wave] = ss;
      __syncthreads();
      float tot = 0.0f;
      for (int w = 0; w < (int)(blockDim.x >> 6); w++) tot += s_ss[w];
      inv = 1.0f / sqrtf(tot / (float)cols + p.norm_eps);
      for (int n = threadIdx.x; n < n4; n += nthr) {
        const float4 g = gsrc[n];
        float4 v = xs4[xs_slot(n >> 4, n & 15)];
        v.x = g.x * (v.x * inv); v.y = g.y * (v.y * inv); v.z = g.z * (v.z * inv); v.w = g.w * (v.w * inv);
        xs4[xs_slot(n >> 4, n & 15)] = v;
      }
    }
    if (!direct) __syncthreads();
    staged = !direct;
  }
  if (act && staged) {
    const int u = sb * 4 + cc;
#pragma unroll
    for (int t = 0; t < 16; t++) {
      const float4 v = xs4[xs_slot(u, t)];
      xv[4 * t] = v.x; xv[4 * t + 1] = v.y; xv[4 * t + 2] = v.z; xv[4 * t + 3] = v.w;
    }
  }
  float sxlo = 0.0f, sxhi = 0.0f;
#pragma unroll
  for (int i = 0; i < 32; i++) { sxlo += xv[i]; sxhi += xv[32 + i]; }

  float ssq_acc = 0.0f;   // squares of the outputs this thread wrote (for the consumer's RMSNorm)
  auto process = [&](Q4kRegs (&cur)[RR], Q4kRegs (&nxt)[RR], int it) {
    const int g = g_first + it * g_stride;
    issue(g + g_stride, nxt);
    float acc[RR];
#pragma unroll
    for (int r = 0; r < RR; r++) acc[r] = 0.0f;
    if (g < n_groups && act) {
#pragma unroll
      for (int r = 0; r < RR; r++) {
        const uint32_t qw[8] = {cur[r].q0.x, cur[r].q0.y, cur[r].q0.z, cur[r].q0.w, cur[r].q1.x, cur[r].q1.y, cur[r].q1.z, cur[r].q1.w};
        float slo = 0.0f, shi = 0.0f;
#pragma unroll
        for (int w = 0; w < 8; w++) {
          // low nibbles as bytes; high nibbles stay in place (16*q per byte, the 1/16 is folded into the scale)
          uint32_t lo = qw[w] & 0x0f0f0f0fu, hi = qw[w] & 0xf0f0f0f0u;
          asm volatile("" : "+v"(lo), "+v"(hi));   // keep the masks whole: each byte converts with one v_cvt_f32_ubyteN
          slo = fmaf(cvt_ub0(lo), xv[4 * w], slo);     slo = fmaf(cvt_ub1(lo), xv[4 * w + 1], slo);
          slo = fmaf(cvt_ub2(lo), xv[4 * w + 2], slo); slo = fmaf(cvt_ub3(lo), xv[4 * w + 3], slo);
          shi = fmaf(cvt_ub0(hi), xv[32 + 4 * w], shi);     shi = fmaf(cvt_ub1(hi), xv[32 + 4 * w + 1], shi);
          shi = fmaf(cvt_ub2(hi), xv[32 + 4 * w + 2], shi); shi = fmaf(cvt_ub3(hi), xv[32 + 4 * w + 3], shi);
        }
        uint32_t sc, mn; q4k_scale_pair(cur[r].h.y, cur[r].h.z, cur[r].h.w, cc, sc, mn);
        const float d = __half2float(__ushort_as_half((unsigned short)(cur[r].h.x & 0xffffu)));
        const float dmin = __half2float(__ushort_as_half((unsigned short)(cur[r].h.x >> 16)));
        acc[r] = d * (cvt_ub0(sc) * slo + (cvt_ub1(sc) * 0.0625f) * shi) - dmin * (cvt_ub0(mn) * sxlo + cvt_ub1(mn) * sxhi);
      }
    }
#pragma unroll
    for (int r = 0; r < RR; r++) acc[r] = wave_sum(acc[r]);   // total in lane 63

    if (nsw > 1) {
      // Slice waves meet every CH row groups: partial sums are parked in LDS (double-buffered by chunk parity), one
      // barrier per chunk, then the lanes of the slice-0 wave finish one output row each.
      const int slot = it % CH, par = (it / CH) & 1;
      if (lane == 63) {
#pragma unroll
        for (int r = 0; r < RR; r++) s_part[par][wave][slot][r] = acc[r];
      }
      if (slot != CH - 1 && it != n_iters - 1) return;
      __syncthreads();
      if (step != 0) return;
      const int n_out = (slot + 1) * (MODE == 1 ? R : RR);
      if (lane >= n_out) return;
      const int sl = lane / (MODE == 1 ? R : RR), r = lane % (MODE == 1 ? R : RR);
      const int gg = g_first + (it - slot + sl) * g_stride;
      if (gg >= n_groups) return;
      const GemvSeg* sg; int row0; locate(gg, sg, row0);
      const int row = row0 + r;
      if (MODE == 0) {
        if (row >= sg->rows) return;
        float v = 0.0f;
        for (int s2 = 0; s2 < nsw; s2++) v += s_part[par][gslot * nsw + s2][sl][r];
        if (sg->bias) v += sg->bias[row];
        v = act_apply(v, p.act);
        const int o = sg->y_off + row;
        if (p.residual) v += p.residual[o];
        p.y[o] = v; ssq_acc = fmaf(v, v, ssq_acc);
      } else {
        if (row >= p.half) return;
        float up = 0.0f, gate = 0.0f;
        for (int s2 = 0; s2 < nsw; s2++) { up += s_part[par][gslot * nsw + s2][sl][2 * r]; gate += s_part[par][gslot * nsw + s2][sl][2 * r + 1]; }
        if (sg->bias) { up += sg->bias[row]; gate += sg->bias[p.half + row]; }
        p.y[sg->y_off + row] = silu_mul(up, gate);
      }
      return;
    }
    if (lane != 63 || g >= n_groups) return;

    const GemvSeg* sg; int row0; locate(g, sg, row0);
    if (MODE == 0) {
#pragma unroll
      for (int r = 0; r < RR; r++) {
        const int row = row0 + r;
        if (row >= sg->rows) break;
        float v = acc[r];
        if (sg->bias) v += sg->bias[row];
        v = act_apply(v, p.act);
        const int o = sg->y_off + row;
        if (p.residual) v += p.residual[o];
        p.y[o] = v; ssq_acc = fmaf(v, v, ssq_acc);
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; r++) {
        const int row = row0 + r;
        if (row >= p.half) break;
        float up = acc[2 * r], gate = acc[2 * r + 1];
        if (sg->bias) { up += sg->bias[row]; gate += sg->bias[p.half + row]; }
        p.y[sg->y_off + row] = silu_mul(up, gate);
      }
    }
  };

  for (int it = 0; it < n_iters; it += 2) {
    process(buf0, buf1, it);
    if (it + 1 < n_iters) process(buf1, buf0, it + 1);
  }

  if (p.ssq_out) {   // per-work-group partial of sum(y^2), summed in a fixed order; unused slots are zeroed by group 0
    __syncthreads();
    const float t = wave_sum(ssq_acc);
    if (lane == 63) s_ss[wave] = t;
    __syncthreads();
    if (threadIdx.x == 0) {
      float tot = 0.0f;
      for (int w = 0; w < (int)(blockDim.x >> 6); w++) tot += s_ss[w];
      p.ssq_out[blockIdx.x] = tot;
    }
    if (blockIdx.x == 0) for (int i = gridDim.x + threadIdx.x; i < SSQ_PARTS; i += blockDim.x) p.ssq_out[i] = 0.0f;
  }
}

// Host launcher.  Returns CAI_ERR_UNSUPPORTED when the shape does not fit this kernel (caller falls back).
int launch_q4k_stream(GemvParams& p, const MultiGemv& m, int swiglu_half, hipStream_t st)
{
  Context& c = ctx();
  const int cols = p.cols, nsb = cols >> 8;
  const int nsw = (nsb + 15) >> 4;          // waves along the columns
  if (nsw > 8) return CAI_ERR_UNSUPPORTED;  // rows longer than 32768 columns
  int gwv = nsw >= 4 ? 1 : (4 / nsw);       // row groups in flight per work-group: keep 4..8 waves per group
  int64_t total = 0;
  for (int i = 0; i < m.n; i++) total += swiglu_half ? swiglu_half : m.rows[i];
  const int waves_per_wg = nsw * gwv;
  // resident work-groups: ~12 waves per CU (VGPR budget of this kernel allows 3 per SIMD)
  int wg_per_cu = 12 / waves_per_wg; if (wg_per_cu < 1) wg_per_cu = 1;
  if (!(gwv == 1 && !(p.norm_gain && !p.ssq_in))) { const int lds_fit = (int)((160 * 1024 - 4096) / ((size_t)((cols + 1023) / 1024 * 1024) * 4 + 1024)); if (wg_per_cu > lds_fit) wg_per_cu = lds_fit < 1 ? 1 : lds_fit; }
  const int max_wgs = c.n_cu * wg_per_cu;
  int R = 1;
  if (!swiglu_half && total >= (int64_t)max_wgs * gwv * 4) R = 2;
  int cum = 0;
  for (int i = 0; i < m.n; i++) {
    const int64_t rows = swiglu_half ? swiglu_half : m.rows[i];
    cum += (int)((rows + R - 1) / R);
    p.seg[i].grp_end = cum;
  }
  const int grid = std::min(std::min((cum + gwv - 1) / gwv, max_wgs), SSQ_PARTS);
  const size_t lds = gwv == 1 && !(p.norm_gain && !p.ssq_in) ? 0 : (size_t)((cols + 1023) / 1024 * 1024) * 4;
  static bool attr_done = false;
  if (!attr_done) {
    const int big = 160 * 1024 - 2048;
    (void)hipFuncSetAttribute((const void*)gemv_q4k_stream<1, 1, false>, hipFuncAttributeMaxDynamicSharedMemorySize, big);
    (void)hipFuncSetAttribute((const void*)gemv_q4k_stream<2, 0, true>, hipFuncAttributeMaxDynamicSharedMemorySize, big);
    (void)hipFuncSetAttribute((const void*)gemv_q4k_stream<1, 0, true>, hipFuncAttributeMaxDynamicSharedMemorySize, big);
    (void)hipFuncSetAttribute((const void*)gemv_q4k_stream<2, 0, false>, hipFuncAttributeMaxDynamicSharedMemorySize, big);
    (void)hipFuncSetAttribute((const void*)gemv_q4k_stream<1, 0, false>, hipFuncAttributeMaxDynamicSharedMemorySize, big);
    attr_done = true;
  }
  const dim3 block(64 * waves_per_wg);
  if (swiglu_half) hipLaunchKernelGGL((gemv_q4k_stream<1, 1, false>), dim3(grid), block, lds, st, p, cum, nsw, gwv);
  else if (m.n > 1) {
    if (R == 2) hipLaunchKernelGGL((gemv_q4k_stream<2, 0, true>), dim3(grid), block, lds, st, p, cum, nsw, gwv);
    else hipLaunchKernelGGL((gemv_q4k_stream<1, 0, true>), dim3(grid), block, lds, st, p, cum, nsw, gwv);
  } else {
    if (R == 2) hipLaunchKernelGGL((gemv_q4k_stream<2, 0, false>), dim3(grid), block, lds, st, p, cum, nsw, gwv);
    else hipLaunchKernelGGL((gemv_q4k_stream<1, 0, false>), dim3(grid), block, lds, st, p, cum, nsw, gwv);
  }
  return CAI_OK;
}

}  // namespace cai
