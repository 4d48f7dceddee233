// Multi-token (prompt) linear layer on the matrix cores for the 32-weight block types, Q8_0 and Q4_0 (one f16 scale per
// block: neural/neuralgguf.pas:389-441, 811-845; resident as a quants plane and a scales plane), dense or grouped by
// expert for a mixture-of-experts prompt (wiring: neural/neuralpretrained.pas:15331-15388).
//
// Accuracy contract as for the Q4_K prompt kernel: the result equals single-token linear layers to fp32 level.  The codes
// (signed bytes, nibble - 8) are exact in f16; an activation is a power-of-two scaled pair of halfs hi + lo (22 bits);
// products accumulate in fp32 on v_mfma_f32_32x32x16_f16; the block scale d multiplies the block's sum in fp32.
//
// d belongs to a weight ROW and a block, so the weights are the B operand (columns of the result = 32 weight rows) and the
// activations the A operand (rows = 32 tokens): lane (n, kg) then holds 16 results of ONE weight row n and d is a value it
// loaded itself - 16 FMAs fold a block's 32 x 32 sums into the running result, no exchange through LDS.  The order of the
// contraction index inside a block is free as long as both operands agree: a lane takes a CONTIGUOUS piece of each block
// (Q8_0: bytes 16 kg .. + 15, two steps of 8; Q4_0: bytes 8 kg .. + 7, low nibbles = weights 8 kg .. + 7 then high nibbles
// = weights 16 + 8 kg .. + 7), so the two lanes of a row read whole 32- / 16-byte blocks and a row's 256 columns are one
// contiguous run.
//
// Work-group: 4 waves x RT row tiles of 32 rows, TT * 32 tokens, 256 columns (8 blocks) per step staged in LDS; with RT = 2
// an activation operand (1 KB of LDS traffic per wave and instruction) feeds two MFMAs.  The next step's weights are
// requested before the current one is consumed.
#include "cai_internal.hpp"
#include "cai_gemv_common.hpp"
#include <algorithm>

namespace cai {

namespace {

typedef _Float16 half2_b __attribute__((ext_vector_type(2)));
typedef _Float16 half8_b __attribute__((ext_vector_type(8)));
typedef float float16_b __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_b __attribute__((ext_vector_type(4)));   // (arrays of HIP's uint4 struct end up in scratch memory)

constexpr int BL_LDX = 264;   // halfs per staged token row: 256 + pad (row stride = 4 banks mod 64: conflict-free 16-byte reads)

struct BlkGemmParams {
  const uint8_t* q; const uint8_t* d; const float* bias;
  int rows, cols;                       // rows of ONE matrix (of one expert's window for a bank)
  const _Float16* xhi; const _Float16* xlo; const float* sinv;   // activation planes [x row][cols], scale per x row
  int n_tok;
  float* y; int64_t y_stride; const float* residual;
  int n_row_groups, n_tok_tiles;
  // grouped by expert: a table of token tiles built on the device (expert, first sorted position, count; count 0 = unused)
  const int32_t* tile_tab; const int32_t* perm;   // perm: sorted position -> slot (token * top_k + rank)
  int x_div;                            // activation row of a slot = slot / x_div; result row = slot
  int64_t expert_rows;
  // dense launches: up to two more matrices of the same type and width (q | k | v) - row groups [seg_end[i], ...) belong to
  // matrix i + 1, whose rows land y_off2[i] columns into a y row
  int n_seg; int seg_end[2];
  const uint8_t* q2[2]; const uint8_t* d2[2]; const float* bias2[2]; int rows2[2]; int y_off2[2];
};

// eight codes (two dwords) -> eight exact halfs.  Q8_0: signed bytes; Q4_0: (nibble - 8), low or high nibbles of the bytes
template <int QT>
__device__ __forceinline__ half8_b codes8(uint32_t w0, uint32_t w1, int high)
{
  uint32_t a, b; _Float16 off;
  if (QT == CAI_Q8_0) { a = w0 ^ 0x80808080u; b = w1 ^ 0x80808080u; off = (_Float16)(-1152.0f); }   // byte + 128 as 1024 + u, minus 1152
  else { a = (high ? (w0 >> 4) : w0) & 0x0f0f0f0fu; b = (high ? (w1 >> 4) : w1) & 0x0f0f0f0fu; off = (_Float16)(-1032.0f); }
  const half2_b o2 = {off, off};
  const half2_b h0 = __builtin_bit_cast(half2_b, __builtin_amdgcn_perm(0x64646464u, a, 0x04010400u)) + o2;
  const half2_b h1 = __builtin_bit_cast(half2_b, __builtin_amdgcn_perm(0x64646464u, a, 0x04030402u)) + o2;
  const half2_b h2 = __builtin_bit_cast(half2_b, __builtin_amdgcn_perm(0x64646464u, b, 0x04010400u)) + o2;
  const half2_b h3 = __builtin_bit_cast(half2_b, __builtin_amdgcn_perm(0x64646464u, b, 0x04030402u)) + o2;
  return half8_b{h0.x, h0.y, h1.x, h1.y, h2.x, h2.y, h3.x, h3.y};
}

}  // namespace

template <int QT, int TT, int RT>
__global__ __launch_bounds__(256, 2) void gemm_blk_pf(const BlkGemmParams p)
{
  extern __shared__ __align__(16) unsigned char bl_smem[];
  constexpr int NTOK = TT * 32;
  _Float16* xs_hi = reinterpret_cast<_Float16*>(bl_smem);            // [NTOK][BL_LDX]
  _Float16* xs_lo = xs_hi + NTOK * BL_LDX;
  __shared__ int s_xrow[NTOK], s_yrow[NTOK];
  __shared__ float s_sinv[NTOK];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, kg = lane >> 5;
  int rg, ttile, first, n_here, expert = 0;
  if (p.tile_tab) {
    ttile = blockIdx.x / p.n_row_groups; rg = blockIdx.x % p.n_row_groups;
    expert = p.tile_tab[3 * ttile]; first = p.tile_tab[3 * ttile + 1]; n_here = p.tile_tab[3 * ttile + 2];
    if (n_here <= 0) return;            // (uniform: the whole work-group leaves)
  } else {
    // linear id = rg_lo + 8 * (tt + n_tok_tiles * rg_hi): the token tiles of a row group share id mod 8, i.e. one XCD and its L2
    const int L = blockIdx.x;
    rg = (L & 7) + 8 * ((L >> 3) / p.n_tok_tiles); ttile = (L >> 3) % p.n_tok_tiles;
    if (rg >= p.n_row_groups) return;
    first = ttile * NTOK; n_here = min(NTOK, p.n_tok - first);
  }
  if (threadIdx.x < NTOK) {
    const int m = min((int)threadIdx.x, n_here - 1);     // rows past the end repeat the last token; their results are not written
    int xr, yr;
    if (p.perm) { const int slot = p.perm[first + m]; xr = slot / p.x_div; yr = slot; }
    else { xr = yr = first + m; }
    s_xrow[threadIdx.x] = xr; s_yrow[threadIdx.x] = yr; s_sinv[threadIdx.x] = p.sinv[xr];
  }
  const uint8_t* qbase = p.q; const uint8_t* dbase = p.d; const float* bias = p.bias; int rows = p.rows, yo = 0, rgl = rg;   // this work-group's matrix (uniform)
  if (p.n_seg > 1 && rg >= p.seg_end[0]) { qbase = p.q2[0]; dbase = p.d2[0]; bias = p.bias2[0]; rows = p.rows2[0]; yo = p.y_off2[0]; rgl = rg - p.seg_end[0]; }
  if (p.n_seg > 2 && rg >= p.seg_end[1]) { qbase = p.q2[1]; dbase = p.d2[1]; bias = p.bias2[1]; rows = p.rows2[1]; yo = p.y_off2[1]; rgl = rg - p.seg_end[1]; }
  const int R0 = (rgl * 4 + wave) * 32 * RT;
  const int K = p.cols, nb32 = K >> 5, nsb = (K + 255) >> 8;
  constexpr int BQ = QT == CAI_Q8_0 ? 32 : 16;          // quant bytes per block
  const int64_t bank_row = (int64_t)expert * p.expert_rows;
  const uint8_t* qrow[RT]; const uint16_t* drow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++) {
    const int64_t r = bank_row + min(R0 + 32 * rt + n, rows - 1);     // tail rows: re-read the last row, not written
    qrow[rt] = qbase + r * (int64_t)nb32 * BQ + (BQ / 2) * kg;
    drow[rt] = reinterpret_cast<const uint16_t*>(dbase) + r * (int64_t)nb32;
  }
  struct WRegs { uint32_t q[4][BQ / 8]; uint32_t d[2]; };               // per row tile: the lane's piece of 4 blocks, their 4 scales
  // unit u = blocks 4 u .. 4 u + 3 of the row.  Loads carry no branch: past the end the last unit / block is fetched again
  // (cache hits, not used), a block at or past the width counts with scale zero.
  auto load_w = [&](int u, WRegs (&w)[RT]) {
    const int uu = min(u, 2 * nsb - 1);
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
#pragma unroll
      for (int b = 0; b < 4; b++) {
        const int bi = min(4 * uu + b, nb32 - 1);
        if constexpr (QT == CAI_Q8_0) {
          const uint4 v = *reinterpret_cast<const uint4*>(qrow[rt] + (int64_t)bi * 32);
          w[rt].q[b][0] = v.x; w[rt].q[b][1] = v.y; w[rt].q[b][2] = v.z; w[rt].q[b][3] = v.w;
        } else {
          const uint2 v = *reinterpret_cast<const uint2*>(qrow[rt] + (int64_t)bi * 16);
          w[rt].q[b][0] = v.x; w[rt].q[b][1] = v.y;
        }
      }
#pragma unroll
      for (int b2 = 0; b2 < 2; b2++) {
        const int b0 = 4 * uu + 2 * b2;
        uint32_t lo = drow[rt][min(b0, nb32 - 1)], hi = drow[rt][min(b0 + 1, nb32 - 1)];
        lo = b0 < nb32 ? lo : 0u; hi = b0 + 1 < nb32 ? hi : 0u;
        w[rt].d[b2] = lo | (hi << 16);
      }
    }
  };

  float16_b Y[RT][TT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++)
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
      for (int v = 0; v < 16; v++) Y[rt][tt][v] = 0.0f;

  const float16_b zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
  // four blocks of the staged 256 columns, starting at block b_first of the tile
  auto compute = [&](const WRegs (&w)[RT], int b_first) {
#pragma unroll
    for (int b = 0; b < 4; b++) {
      half8_b W[RT][2];
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        if constexpr (QT == CAI_Q8_0) { W[rt][0] = codes8<QT>(w[rt].q[b][0], w[rt].q[b][1], 0); W[rt][1] = codes8<QT>(w[rt].q[b][2], w[rt].q[b][3], 0); }
        else { W[rt][0] = codes8<QT>(w[rt].q[b][0], w[rt].q[b][1], 0); W[rt][1] = codes8<QT>(w[rt].q[b][0], w[rt].q[b][1], 1); }
      }
      float16_b C[RT][TT];
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
          // Q8_0: the lane's k of step s are columns 16 kg + 8 s .. of the block; Q4_0: 16 s + 8 kg ..
          const int koff = QT == CAI_Q8_0 ? 16 * kg + 8 * s : 16 * s + 8 * kg;
          const int off = (tt * 32 + n) * BL_LDX + 32 * (b_first + b) + koff;
          const half8_b Ah = *reinterpret_cast<const half8_b*>(xs_hi + off);
          const half8_b Al = *reinterpret_cast<const half8_b*>(xs_lo + off);
#pragma unroll
          for (int rt = 0; rt < RT; rt++) C[rt][tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Ah, W[rt][s], s == 0 ? zero16 : C[rt][tt], 0, 0, 0);
#pragma unroll
          for (int rt = 0; rt < RT; rt++) C[rt][tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(Al, W[rt][s], C[rt][tt], 0, 0, 0);
        }
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        const uint32_t dw = w[rt].d[b >> 1];
        const float dv = __half2float(__ushort_as_half((unsigned short)((b & 1) ? (dw >> 16) : (dw & 0xffffu))));
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
          for (int v = 0; v < 16; v++) Y[rt][tt][v] = fmaf(dv, C[rt][tt][v], Y[rt][tt][v]);
      }
    }
  };

  WRegs wa[RT], wb[RT];
  load_w(0, wa);
  __syncthreads();                         // the row tables
  for (int sb = 0; sb < nsb; sb++) {
    if (sb) __syncthreads();               // the previous step's LDS reads are done
    {
      // thread = (token tq + 8 i, 16-byte chunk); columns at or past the width are staged as zeros
      const int tq = threadIdx.x >> 5, chunk = threadIdx.x & 31;
      const int col = sb * 256 + chunk * 8;
      const bool in = col < K;
      const uint32_t colo = (uint32_t)(in ? col : 0);
      constexpr int SB = TT == 2 ? 2 : 4;
#pragma unroll
      for (int i0 = 0; i0 < NTOK / 8; i0 += SB) {
        u32x4_b vh[SB], vl[SB];
#pragma unroll
        for (int i = 0; i < SB; i++) {
          const int64_t off = (int64_t)s_xrow[tq + 8 * (i0 + i)] * K + colo;
          vh[i] = *reinterpret_cast<const u32x4_b*>(p.xhi + off);
          vl[i] = *reinterpret_cast<const u32x4_b*>(p.xlo + off);
        }
#pragma unroll
        for (int i = 0; i < SB; i++) {
          const u32x4_b z = {0u, 0u, 0u, 0u};
          *reinterpret_cast<u32x4_b*>(xs_hi + (tq + 8 * (i0 + i)) * BL_LDX + chunk * 8) = in ? vh[i] : z;
          *reinterpret_cast<u32x4_b*>(xs_lo + (tq + 8 * (i0 + i)) * BL_LDX + chunk * 8) = in ? vl[i] : z;
        }
      }
    }
    load_w(2 * sb + 1, wb);
    __syncthreads();
    compute(wa, 0);
    load_w(2 * sb + 2, wa);                // the next step's first half is in flight while this step's second half is consumed
    compute(wb, 4);
  }

  // ---- write: the lane holds weight row n of each row tile and tokens 8 g + 4 kg + i of each token tile: the 32 lanes of a
  // half-wave store 32 consecutive outputs of one token row ----
#pragma unroll
  for (int tt = 0; tt < TT; tt++)
#pragma unroll
    for (int g = 0; g < 4; g++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int m = tt * 32 + 8 * g + 4 * kg + i;
        if (m >= n_here) continue;
        const float si = s_sinv[m];
        const int64_t o = (int64_t)s_yrow[m] * p.y_stride;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
          const int row = R0 + 32 * rt + n;
          if (row >= rows) continue;
          float r = Y[rt][tt][4 * g + i] * si;
          if (bias) r += bias[bank_row + row];
          if (p.residual) r += p.residual[o + yo + row];
          p.y[o + yo + row] = r;
        }
      }
}

// ------------------------------------------------------------------------------------------
// Grouping of a prompt's (token, rank) slots by expert: perm lists the slots expert by expert, tile_tab cuts each expert's
// run into token tiles of at most `tile` slots.  One work-group; the order of the slots inside an expert's run depends on
// the arrival of LDS atomics, which does not matter: every result row is computed from its own activation row only.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t* expert, int n_slots, int n_experts, int tile, int max_tiles,
                                                         int32_t* perm, int32_t* tile_tab)
{
  __shared__ int cnt[512], off[513], cur[512];
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) { cnt[e] = 0; cur[e] = 0; }
  __syncthreads();
  for (int s = threadIdx.x; s < n_slots; s += blockDim.x) atomicAdd(&cnt[min(max(expert[s], 0), n_experts - 1)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int o = 0, t = 0;
    for (int e = 0; e < n_experts; e++) {
      off[e] = o;
      for (int k = 0; k < cnt[e]; k += tile, t++) { tile_tab[3 * t] = e; tile_tab[3 * t + 1] = o + k; tile_tab[3 * t + 2] = min(tile, cnt[e] - k); }
      o += cnt[e];
    }
    off[n_experts] = o;
    for (; t < max_tiles; t++) { tile_tab[3 * t] = 0; tile_tab[3 * t + 1] = 0; tile_tab[3 * t + 2] = 0; }
  }
  __syncthreads();
  for (int s = threadIdx.x; s < n_slots; s += blockDim.x) {
    const int e = min(max(expert[s], 0), n_experts - 1);
    perm[off[e] + atomicAdd(&cur[e], 1)] = s;
  }
}

namespace {

template <int QT>
int launch_blk(const BlkGemmParams& p0, int n_tiles_grouped)
{
  BlkGemmParams p = p0;
  const int n_cu = ctx().n_cu;
  static bool attr_done = false;
  if (!attr_done) {
    const void* ks[] = {(const void*)gemm_blk_pf<CAI_Q8_0, 1, 1>, (const void*)gemm_blk_pf<CAI_Q8_0, 1, 2>, (const void*)gemm_blk_pf<CAI_Q8_0, 2, 2>,
                        (const void*)gemm_blk_pf<CAI_Q4_0, 1, 1>, (const void*)gemm_blk_pf<CAI_Q4_0, 1, 2>, (const void*)gemm_blk_pf<CAI_Q4_0, 2, 2>};
    for (const void* k : ks) if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess) (void)hipGetLastError();
    attr_done = true;
  }
  // Tiling: two row tiles per wave (256 rows per work-group) whenever that still gives every CU work; two token tiles on top
  // for long prompts; one row tile for matrices of few rows
  const int tiles32 = p.tile_tab ? n_tiles_grouped : (p.n_tok + 31) / 32;
  int rows_all = p.rows;
  for (int i = 1; i < p.n_seg; i++) rows_all += p.rows2[i - 1];
  const int wgs_rt2 = ((rows_all + 255) / 256) * tiles32;
  int rt = wgs_rt2 >= n_cu ? 2 : 1, tt = 1;
  if (!p.tile_tab && rt == 2 && ((rows_all + 255) / 256) * ((p.n_tok + 63) / 64) >= 2 * n_cu) tt = 2;
  p.n_row_groups = (p.rows + 128 * rt - 1) / (128 * rt);
  for (int i = 1; i < p.n_seg; i++) { p.seg_end[i - 1] = p.n_row_groups; p.n_row_groups += (p.rows2[i - 1] + 128 * rt - 1) / (128 * rt); }   // every matrix starts a row group of its own
  const size_t lds = (size_t)tt * 32 * BL_LDX * 2 * 2;
  int grid;
  if (p.tile_tab) { p.n_tok_tiles = n_tiles_grouped; grid = n_tiles_grouped * p.n_row_groups; }
  else { p.n_tok_tiles = (p.n_tok + tt * 32 - 1) / (tt * 32); grid = 8 * p.n_tok_tiles * ((p.n_row_groups + 7) / 8); }
  hipStream_t st = ctx().stream;
  if (tt == 2) hipLaunchKernelGGL((gemm_blk_pf<QT, 2, 2>), dim3(grid), dim3(256), lds, st, p);
  else if (rt == 2) hipLaunchKernelGGL((gemm_blk_pf<QT, 1, 2>), dim3(grid), dim3(256), lds, st, p);
  else hipLaunchKernelGGL((gemm_blk_pf<QT, 1, 1>), dim3(grid), dim3(256), lds, st, p);
  return CAI_OK;
}

}  // namespace

bool gemm_blk_supported(const cai_qw_s* w) { return (w->qtype == CAI_Q8_0 || w->qtype == CAI_Q4_0) && w->cols % 32 == 0; }

// Dense: y[t][rows] = W x[t] (+ bias) (+ residual) for the n_tok prepared activation rows.
int launch_gemm_blk(const cai_qw_s* w, const _Float16* xhi, const _Float16* xlo, const float* sinv, int n_tok, float* y, int64_t y_stride,
                    const float* residual)
{
  if (!gemm_blk_supported(w)) return set_error(CAI_ERR_UNSUPPORTED, "prompt gemm: weight type %d", w->qtype);
  BlkGemmParams p{};
  p.q = w->data; p.d = w->aux; p.bias = w->bias; p.rows = (int)w->rows; p.cols = (int)w->cols;
  p.xhi = xhi; p.xlo = xlo; p.sinv = sinv; p.n_tok = n_tok; p.y = y; p.y_stride = y_stride; p.residual = residual;
  p.x_div = 1; p.expert_rows = 0;
  return w->qtype == CAI_Q8_0 ? launch_blk<CAI_Q8_0>(p, 0) : launch_blk<CAI_Q4_0>(p, 0);
}

// Up to three matrices of one type and width in one launch: y[t][y_off[i] + r] = (W_i x[t])[r] (+ bias_i)
bool gemm_blk_multi_supported(const cai_qw_s* const* ws, int n_w)
{
  if (n_w < 1 || n_w > 3 || !gemm_blk_supported(ws[0])) return false;
  for (int i = 1; i < n_w; i++) if (ws[i]->qtype != ws[0]->qtype || ws[i]->cols != ws[0]->cols) return false;
  return true;
}
int launch_gemm_blk_multi(const cai_qw_s* const* ws, const int* y_off, int n_w, const _Float16* xhi, const _Float16* xlo, const float* sinv,
                          int n_tok, float* y, int64_t y_stride)
{
  if (!gemm_blk_multi_supported(ws, n_w)) return set_error(CAI_ERR_UNSUPPORTED, "prompt gemm: %d matrices in one launch", n_w);
  const cai_qw_s* w = ws[0];
  BlkGemmParams p{};
  p.q = w->data; p.d = w->aux; p.bias = w->bias; p.rows = (int)w->rows; p.cols = (int)w->cols;
  p.xhi = xhi; p.xlo = xlo; p.sinv = sinv; p.n_tok = n_tok; p.y = y + y_off[0]; p.y_stride = y_stride; p.residual = nullptr;
  p.x_div = 1; p.expert_rows = 0; p.n_seg = n_w;
  for (int i = 1; i < n_w; i++) { p.q2[i - 1] = ws[i]->data; p.d2[i - 1] = ws[i]->aux; p.bias2[i - 1] = ws[i]->bias; p.rows2[i - 1] = (int)ws[i]->rows; p.y_off2[i - 1] = y_off[i] - y_off[0]; }
  return w->qtype == CAI_Q8_0 ? launch_blk<CAI_Q8_0>(p, 0) : launch_blk<CAI_Q4_0>(p, 0);
}

// Token tiles of the grouped launches: every expert may end with a partial tile
int moe_group_max_tiles(int n_slots, int n_experts) { return (n_slots + 31) / 32 + n_experts; }

int launch_moe_group(const int32_t* expert, int n_slots, int n_experts, int32_t* perm, int32_t* tile_tab)
{
  if (n_experts > 512) return set_error(CAI_ERR_UNSUPPORTED, "moe grouping: %d experts (up to 512)", n_experts);
  hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 0, ctx().stream, expert, n_slots, n_experts, 32, moe_group_max_tiles(n_slots, n_experts), perm, tile_tab);
  return CAI_OK;
}

// Grouped: slot s (a token's rank-th expert) takes activation row s / x_div through the rows [e * expert_rows, + expert_rows)
// of the bank, e the slot's expert; the result goes to row s of y.
int launch_gemm_blk_grouped(const cai_qw_s* bank, int64_t expert_rows, const _Float16* xhi, const _Float16* xlo, const float* sinv, int x_div,
                            int n_slots, int n_experts, const int32_t* perm, const int32_t* tile_tab, float* y, int64_t y_stride)
{
  if (!gemm_blk_supported(bank)) return set_error(CAI_ERR_UNSUPPORTED, "grouped prompt gemm: weight type %d", bank->qtype);
  if (expert_rows <= 0 || bank->rows != expert_rows * n_experts) return set_error(CAI_ERR_INVALID, "grouped prompt gemm: bank of %lld rows is not %d windows of %lld", (long long)bank->rows, n_experts, (long long)expert_rows);
  BlkGemmParams p{};
  p.q = bank->data; p.d = bank->aux; p.bias = bank->bias; p.rows = (int)expert_rows; p.cols = (int)bank->cols;
  p.xhi = xhi; p.xlo = xlo; p.sinv = sinv; p.n_tok = n_slots; p.y = y; p.y_stride = y_stride; p.residual = nullptr;
  p.tile_tab = tile_tab; p.perm = perm; p.x_div = x_div; p.expert_rows = expert_rows;
  const int tiles = moe_group_max_tiles(n_slots, n_experts);
  return bank->qtype == CAI_Q8_0 ? launch_blk<CAI_Q8_0>(p, tiles) : launch_blk<CAI_Q4_0>(p, tiles);
}

}  // namespace cai
