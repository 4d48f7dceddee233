// Small-batch (2..8 tokens per pass) Q4_K linear layer on the matrix cores of gfx950: the decode step of a few sequences.
//
// At batch 1 the layer is a matrix-vector product and the VALU keeps up with HBM; at batch b the same weights serve
// b activations, so the contraction goes to v_mfma_f32_16x16x32_f16 while the weights are still streamed once.
//   * A operand = sc_j * q, an integer <= 63 * 15 and therefore EXACT in f16: the 6-bit sub-block scale is folded into
//     the nibble with one packed fma ((1024 + q) * sc - 1024 * sc, every term exact), so the matrix cores accumulate
//     across a whole 256-weight super-block and the float scale d is applied once per super-block, not per 32 weights;
//   * B operand = the activations of up to 8 tokens, scaled per (token, 256-block) by a power of two and split hi + lo
//     into two f16 (22 significant bits): 8 hi + 8 lo = the 16 columns of the MFMA tile;
//   * the -dmin * mn_j * sum_{k in j} x_k term is one more MFMA per row set and super-block (k = the 8 sub-blocks).
//   Y[t][r] = sum_sb sinv[t][sb] * ( d * P_main - 32 dmin * P_min )   (Q4_K: neural/neuralgguf.pas:472-514)
//
// Work layout: grid = (row groups, K slices).  A work-group stages ITS slice of the activations (up to 4 super-blocks)
// in LDS once, then its 4 waves walk 32-row tiles independently - no barrier after the staging, weights of the next
// two (tile, super-block) items always in flight.  Each slice writes a partial result; the consumer (next activation
// pre-pass, SwiGLU, or a plain reduction) adds the slices in a fixed order.  Token RMSNorm factors out of the product:
// the pre-pass stores g*x and per-block sums of squares, the consumer multiplies by 1/rms (neural/neural.cl:1047-1085).
#include "cai_internal.hpp"
#include "cai_gemv_common.hpp"
#include <algorithm>

namespace cai {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int NB_LDX = 264;      // halfs per staged activation column: 256 + pad (stride = 4 banks mod 64: 16-byte reads of 16 columns tile the banks)
constexpr int NB_SC = 16;        // staged columns: 8 tokens x {hi, lo}
constexpr int NB_TK = 8;         // tokens per matrix-core group (8 hi + 8 lo = the 16 rows of an MFMA operand) and per pass of most kernels
constexpr int NB_TMAX = 16;      // tokens per pass at most (the Q6_K kernel takes two groups; four spill its accumulators); the workspace holds this many
constexpr int NB_SMAX = 5;       // super-blocks per K slice at most (LDS: 8.6 KB each, and three work-groups share a CU)

struct NbSeg { const uint8_t* w; const uint8_t* aux; const uint8_t* aux2; const float* bias; const float* row_scale; int rows; int y_off; int tile_end; };   // aux: block scales plane (Q8_0 / Q4_0 / Q6_K); aux2: Q6_K plane of d; row_scale: per-row int8 matrices; tile_end: cumulative 32-row tiles

struct NbParams {
  NbSeg seg[3]; int n_seg;                      // up to three matrices of equal width share one launch (q | k | v)
  int n_tiles;
  int cols;
  const _Float16* xhi; const _Float16* xlo;     // [token][cols]
  const _Float16* sxhi; const _Float16* sxlo;   // [token][cols/32]: (sum of the 32-block) * s / 32, split hi + lo
  const float* sinvb;                           // [token][cols/256] 1 / s of the (token, 256-block)
  int n_tok;
  float* part; int64_t part_stride;             // part[(slice*n_tok + t)*part_stride + y_off + row]
  int sb_per_slice;
  int tile_stride;                              // tiles between two tiles of the same wave (= 4 * gridDim.x)
};

__device__ __forceinline__ half4_t bytes_to_half4(uint32_t t)
{
  // four bytes (0..255) -> four exact halfs 1024 + b (the byte becomes the low mantissa bits of 0x6400 = 1024.0)
  const uint32_t p01 = __builtin_amdgcn_perm(0x64646464u, t, 0x04010400u);
  const uint32_t p23 = __builtin_amdgcn_perm(0x64646464u, t, 0x04030402u);
  const half2_t a = __builtin_bit_cast(half2_t, p01), b = __builtin_bit_cast(half2_t, p23);
  return half4_t{a.x, a.y, b.x, b.y};
}

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// eight nibbles (one per byte of lo, hi) times the sub-block scale -> the eight exact halfs sc * q
__device__ __forceinline__ half8_t nibbles_times_scale(uint32_t lo, uint32_t hi, half2_t s2, half2_t c2)
{
  const half2_t a0 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, lo, 0x04010400u)), s2, c2);   // (1024 + q) * sc - 1024 * sc
  const half2_t a1 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, lo, 0x04030402u)), s2, c2);
  const half2_t a2 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, hi, 0x04010400u)), s2, c2);
  const half2_t a3 = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, hi, 0x04030402u)), s2, c2);
  return half8_t{a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
}

// v_mfma_f32_16x16x32_f16: lane (m = lane % 16, kg = lane / 16) supplies 8 consecutive k of row m (A) / column m (B);
// the 16 x 16 result has rows 4 kg .. 4 kg + 3 of column m in this lane.  Here a tile is 32 weight rows = two row sets,
// the 16 columns are 8 tokens x {hi, lo}.  The order of k inside a super-block is free (both operands follow it), so it is
// chosen for the requests: the four kg lanes of a row ask for 64 CONTIGUOUS quant bytes per request (bytes 16 kg .. + 15,
// then 64 + 16 kg .. + 15), which touches each 64-byte sector of the 144-byte blocks once per request; with 32 contiguous
// bytes per lane every request touched the pieces of all sectors of a block.  Lane kg therefore owns weights
// 16 (kg & 1) .. + 15 of sub-blocks 2 g, 2 g + 1 (low, high nibbles) for g = kg / 2 and for g = 2 + kg / 2.
// QT = CAI_Q5_K: the same walk over 176-byte super-blocks (neural/neuralgguf.pas:516-587): header as Q4_K, then the 32-byte plane of
// fifth bits (bit j of byte i belongs to weight i of sub-block j), then the nibbles; sc * (nibble | bit << 4) <= 63 * 31 stays exact in f16.
template <int QT>
__global__ __launch_bounds__(256, 2) void gemm_q4k_nb(const _Float16* hxhi, const _Float16* hxlo, const _Float16* hsxhi, const _Float16* hsxlo, const float* hsinvb, const int hcols, const int hntok, const int hS, const int hntiles, const NbParams p)
{
  constexpr int BB = QT == CAI_Q5_K ? 176 : 144, QOFF = QT == CAI_Q5_K ? 48 : 16;
  extern __shared__ __align__(16) unsigned char nb_smem[];
  const int S = hS;
  _Float16* xs = reinterpret_cast<_Float16*>(nb_smem);              // [S][16][NB_LDX]
  _Float16* sxs = xs + S * NB_SC * NB_LDX;                           // [S][16][8]
  float* sinv_s = reinterpret_cast<float*>(sxs + S * NB_SC * 8);     // [S][8]
  float* s_d = sinv_s + S * NB_TK;                                   // [4 waves][2][32]: d, 32*dmin per row
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: segment lookups and loop bounds stay scalar
  const int n = lane & 15, kg = lane >> 4;
  const int K = hcols, nsb = K >> 8, nb32 = K >> 5;
  const int slice = blockIdx.y, sb0 = slice * S, nS = min(S, nsb - sb0);
  const int64_t row_bytes = (int64_t)nsb * BB;
  const int tile0 = blockIdx.x * 4 + wave;
  const int n_it = tile0 < hntiles ? (hntiles - tile0 + p.tile_stride - 1) / p.tile_stride : 0;
  const int nq = n_it * nS;                      // (tile, super-block) items of this wave

  struct WRegs { uint4 h[2], q[2][2], e[QT == CAI_Q5_K ? 2 : 1][2]; };   // e: Q5_K's bit plane (all 32 bytes: every lane needs its two bits of each)
  auto locate = [&](int tile, const NbSeg*& sg, int& R0) {
    int sgi = 0, t0 = 0;
    if (p.n_seg > 1 && tile >= p.seg[0].tile_end) { sgi = 1; t0 = p.seg[0].tile_end; }
    if (p.n_seg > 2 && tile >= p.seg[1].tile_end) { sgi = 2; t0 = p.seg[1].tile_end; }
    sg = &p.seg[sgi]; R0 = (tile - t0) * 32;
  };
  // weights of item q: for rows R0 + n and R0 + 16 + n the header and this lane's 32 quant bytes
  // Loads are never conditional: past the wave's last item the last one is fetched again (a cache hit).  A load under a
  // branch would make the compiler wait for ALL outstanding loads at every join.
  auto load_w = [&](int q, WRegs& r) {
    const int qc = max(min(q, nq - 1), 0);
    const int tile = min(tile0 + (qc / nS) * p.tile_stride, hntiles - 1), sb = sb0 + qc % nS;
    const NbSeg* sg; int R0; locate(tile, sg, R0);
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      const uint8_t* blk = sg->w + (int64_t)min(R0 + 16 * hh + n, sg->rows - 1) * row_bytes + (int64_t)sb * BB;   // tail rows: re-read the last row
      r.h[hh] = *reinterpret_cast<const uint4*>(blk);
      r.q[hh][0] = *reinterpret_cast<const uint4*>(blk + QOFF + 16 * kg);
      r.q[hh][1] = *reinterpret_cast<const uint4*>(blk + QOFF + 64 + 16 * kg);
      if constexpr (QT == CAI_Q5_K) { r.e[hh][0] = *reinterpret_cast<const uint4*>(blk + 16); r.e[hh][1] = *reinterpret_cast<const uint4*>(blk + 32); }
    }
  };
  WRegs wa, wb, wc;

  // ---- stage this slice of the activations: nS x 16 columns x 256 halfs, block sums, block scales ----
  // Requests return in the order they were issued: the first batch of activation requests goes out BEFORE the first weight
  // requests (which do not depend on the staging), so that the staged values do not queue behind the first burst of weights.
  // All requests of a thread are issued before the first value is stored (four at a time for the big array): one memory
  // round trip per four chunks instead of one per chunk.  Requests are unconditional (clamped token), absent tokens zeroed.
  {
    const int n_sx = nS * NB_SC;                   // small arrays: one thread per (super-block, column)
    const bool sx_on = (int)threadIdx.x < n_sx;
    const int sx_i = min((int)threadIdx.x, n_sx - 1), sx_col = sx_i % NB_SC, sx_s = sx_i / NB_SC, sx_tok = sx_col % NB_TK;
    const int sx_tc = min(sx_tok, hntok - 1);
    const uint4 sxv = *reinterpret_cast<const uint4*>(((sx_col / NB_TK) ? hsxlo : hsxhi) + (int64_t)sx_tc * nb32 + (sb0 + sx_s) * 8);
    const float siv = hsinvb[(int64_t)sx_tc * nsb + sb0 + sx_s];
    const int total = nS * NB_SC * 32;
    for (int base = 0; base < total; base += 4 * 256) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int idx = min(base + u * 256 + (int)threadIdx.x, total - 1);
        const int chunk = idx & 31, col = (idx >> 5) % NB_SC, s = (idx >> 5) / NB_SC, tok = min(col % NB_TK, hntok - 1);
        v[u] = *reinterpret_cast<const uint4*>(((col / NB_TK) ? hxlo : hxhi) + (int64_t)tok * K + (sb0 + s) * 256 + chunk * 8);
      }
      if (base == 0) { load_w(0, wa); load_w(1, wb); }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int idx = base + u * 256 + (int)threadIdx.x;
        if (idx < total) {
          const int chunk = idx & 31, col = (idx >> 5) % NB_SC, s = (idx >> 5) / NB_SC;
          *reinterpret_cast<uint4*>(xs + (s * NB_SC + col) * NB_LDX + chunk * 8) = (col % NB_TK) < hntok ? v[u] : make_uint4(0, 0, 0, 0);
        }
      }
    }
    if (sx_on) {
      *reinterpret_cast<uint4*>(sxs + sx_i * 8) = sx_tok < hntok ? sxv : make_uint4(0, 0, 0, 0);
      if (sx_col < NB_TK) sinv_s[sx_s * NB_TK + sx_tok] = sx_tok < hntok ? siv : 0.0f;
    }
  }
  __syncthreads();

  float acc[2][4];
  const _Float16 k1024 = (_Float16)1024.0f, kz = (_Float16)0.0f;

  auto compute = [&](const WRegs& r, int q) {
    const int s = q % nS;
    if (s == 0) {
#pragma unroll
      for (int hh = 0; hh < 2; hh++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[hh][i] = 0.0f;
    }
    float4_t C[2], Cm[2];
    half2_t s2[2][4], c2[2][4];
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      // 6-bit scales / mins (neural/neuralgguf.pas:448-464), one per byte: sub-blocks 0..3 and 4..7; this lane's two
      const uint4 h = r.h[hh];
      const uint32_t sc_lo = h.y & 0x3f3f3f3fu, sc_hi = (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u);
      const uint32_t mn_lo = h.z & 0x3f3f3f3fu, mn_hi = ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u);
      // the lane's quant bytes are those of byte groups kg / 2 (first request) and 2 + kg / 2 (second): sub-blocks
      // 2 (kg / 2), + 1 (low, high nibbles) and 4 + 2 (kg / 2), + 1; the min term below keeps sub-blocks 2 kg, 2 kg + 1
      const uint32_t scq[2] = {sc_lo >> (16 * (kg >> 1)), sc_hi >> (16 * (kg >> 1))};
      const uint32_t mnp = ((kg & 2) ? mn_hi : mn_lo) >> (16 * (kg & 1));
      const half2_t mnh = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, mnp, 0x04010400u)) - half2_t{k1024, k1024};
#pragma unroll
      for (int c = 0; c < 2; c++) {
        const half2_t sch = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, scq[c], 0x04010400u)) - half2_t{k1024, k1024};
        s2[hh][2 * c] = half2_t{sch.x, sch.x}; s2[hh][2 * c + 1] = half2_t{sch.y, sch.y};
        c2[hh][2 * c] = half2_t{(_Float16)(-1024.0f) * sch.x, (_Float16)(-1024.0f) * sch.x};   // exact: a multiple of 1024 below 65504
        c2[hh][2 * c + 1] = half2_t{(_Float16)(-1024.0f) * sch.y, (_Float16)(-1024.0f) * sch.y};
      }
      if (kg == 0) {
        const float d = __half2float(__ushort_as_half((unsigned short)(h.x & 0xffffu)));
        const float dmin = __half2float(__ushort_as_half((unsigned short)(h.x >> 16)));
        s_d[(wave * 2 + 0) * 32 + 16 * hh + n] = d; s_d[(wave * 2 + 1) * 32 + 16 * hh + n] = dmin * 32.0f;
      }
      // - dmin * mn_j * (sum of the sub-block's activations): k = this lane's two sub-blocks, the other six k stay zero
      const half2_t bm = *reinterpret_cast<const half2_t*>(sxs + (s * NB_SC + n) * 8 + 2 * kg);
      const half8_t Am = {mnh.x, mnh.y, kz, kz, kz, kz, kz, kz}, Bm = {bm.x, bm.y, kz, kz, kz, kz, kz, kz};
      const float4_t z4 = {0.0f, 0.0f, 0.0f, 0.0f};
      Cm[hh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Am, Bm, z4, 0, 0, 0);
      C[hh] = z4;
    }
    // step t = 4 c + 2 nib + j: request c, low or high nibbles, bytes 8 j .. 8 j + 7 of the lane's 16 = weights
    // 16 (kg & 1) + 8 j .. + 7 of sub-block 2 (kg / 2 + 2 c) + nib
    const _Float16* xcol = xs + (s * NB_SC + n) * NB_LDX + 64 * (kg >> 1) + 16 * (kg & 1);
    uint4 ee[2];
    if constexpr (QT == CAI_Q5_K) {
#pragma unroll
      for (int hh = 0; hh < 2; hh++) ee[hh] = (kg & 1) ? r.e[hh][1] : r.e[hh][0];   // plane bytes 16 (kg & 1) .. + 15
    }
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const int c = t >> 2, nib = (t >> 1) & 1, j = t & 1;
      const half8_t B = *reinterpret_cast<const half8_t*>(xcol + 128 * c + 32 * nib + 8 * j);
#pragma unroll
      for (int hh = 0; hh < 2; hh++) {
        const uint4& qq = r.q[hh][c];
        const uint32_t d0 = j ? qq.z : qq.x, d1 = j ? qq.w : qq.y;
        uint32_t lo = nib ? ((d0 >> 4) & 0x0f0f0f0fu) : (d0 & 0x0f0f0f0fu);
        uint32_t hi = nib ? ((d1 >> 4) & 0x0f0f0f0fu) : (d1 & 0x0f0f0f0fu);
        if constexpr (QT == CAI_Q5_K) {   // bit (sub-block) of the plane bytes of these weights
          const uint32_t e0 = j ? ee[hh].z : ee[hh].x, e1 = j ? ee[hh].w : ee[hh].y;
          const int bit = 2 * ((kg >> 1) + 2 * c) + nib;
          lo |= ((e0 >> bit) & 0x01010101u) << 4; hi |= ((e1 >> bit) & 0x01010101u) << 4;
        }
        const half8_t A = nibbles_times_scale(lo, hi, s2[hh][2 * c + nib], c2[hh][2 * c + nib]);
        C[hh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, C[hh], 0, 0, 0);
      }
    }
    const float si = sinv_s[s * NB_TK + (n & (NB_TK - 1))];
    __builtin_amdgcn_wave_barrier();   // s_d was written by this wave's own lanes above; LDS operations of a wave complete in order
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      const float4 d4 = *reinterpret_cast<const float4*>(&s_d[(wave * 2 + 0) * 32 + 16 * hh + 4 * kg]);
      const float4 m4 = *reinterpret_cast<const float4*>(&s_d[(wave * 2 + 1) * 32 + 16 * hh + 4 * kg]);
      acc[hh][0] += si * (d4.x * C[hh][0] - m4.x * Cm[hh][0]);
      acc[hh][1] += si * (d4.y * C[hh][1] - m4.y * Cm[hh][1]);
      acc[hh][2] += si * (d4.z * C[hh][2] - m4.z * Cm[hh][2]);
      acc[hh][3] += si * (d4.w * C[hh][3] - m4.w * Cm[hh][3]);
    }
    __builtin_amdgcn_wave_barrier();
    if (s != nS - 1) return;
    // ---- the slice's contribution of this tile: column t (hi) + column 8 + t (lo); lane t keeps 2 runs of 4 rows ----
    const int tile = tile0 + (q / nS) * p.tile_stride;
    const NbSeg* sg; int R0; locate(tile, sg, R0);
    const int tok = n & (NB_TK - 1);
    float tot[2][4];
#pragma unroll
    for (int hh = 0; hh < 2; hh++)
#pragma unroll
      for (int i = 0; i < 4; i++) tot[hh][i] = acc[hh][i] + __shfl_xor(acc[hh][i], NB_TK, 64);
    if (n < NB_TK && tok < hntok) {
      float* dst = p.part + ((int64_t)slice * hntok + tok) * p.part_stride + sg->y_off;
#pragma unroll
      for (int hh = 0; hh < 2; hh++) {
        const int row = R0 + 16 * hh + 4 * kg;
        if (row + 3 < sg->rows && ((sg->y_off + row) & 3) == 0) *reinterpret_cast<float4*>(dst + row) = make_float4(tot[hh][0], tot[hh][1], tot[hh][2], tot[hh][3]);
        else {
#pragma unroll
          for (int i = 0; i < 4; i++) if (row + i < sg->rows) dst[row + i] = tot[hh][i];
        }
      }
    }
  };

  for (int q = 0; q < nq; q += 3) {
    load_w(q + 2, wc); compute(wa, q);
    load_w(q + 3, wa); if (q + 1 < nq) compute(wb, q + 1);
    load_w(q + 4, wb); if (q + 2 < nq) compute(wc, q + 2);
  }
}

// ------------------------------------------------------------------------------------------
// Q8_0 / Q4_0 (32-weight blocks, one f16 scale each: neural/neuralgguf.pas:389-441), stored as a quants plane and a
// scales plane.  The block scale d belongs to a weight ROW, so here the roles of the operands are swapped: the
// activations are the A operand (16 rows = 8 tokens x {hi, lo}) and 16 weight rows are the B operand.  A lane then
// holds, for ONE weight row (lane % 16), the results of rows 4 kg .. 4 kg + 3 = four tokens - and d of its own row
// is a value it loaded itself: result += d * (one MFMA over the 32 weights of the block), no exchange through LDS.
// The codes are exact in f16: Q8_0 signed bytes, Q4_0 nibble - 8.  Columns are walked in groups of 8 blocks (the
// granularity of the activation scales); a row's last group may be short (width % 256 != 0): the block index is
// clamped, the staged activations beyond the width are zero and the scale of such a block counts as zero.
// ------------------------------------------------------------------------------------------
struct __attribute__((aligned(4))) Dwords4 { uint32_t x, y, z, w; };   // scale rows are 2-byte items: 4-byte alignment only

template <int QT> __device__ __forceinline__ half8_t codes_to_half8(uint32_t w0, uint32_t w1)
{
  uint32_t a, b; _Float16 off;
  if (QT == CAI_Q8_0 || QT == CAI_I8ROW) { a = w0 ^ 0x80808080u; b = w1 ^ 0x80808080u; off = (_Float16)(-1152.0f); }   // byte + 128, then 1024 + .. - 1152
  else { a = w0 & 0x0f0f0f0fu; b = (w0 >> 4) & 0x0f0f0f0fu; off = (_Float16)(-1032.0f); }           // elements e and 16 + e of the block
  const half2_t o2 = {off, off};
  const half2_t h0 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, a, 0x04010400u)) + o2;
  const half2_t h1 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, a, 0x04030402u)) + o2;
  const half2_t h2 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, b, 0x04010400u)) + o2;
  const half2_t h3 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, b, 0x04030402u)) + o2;
  return half8_t{h0.x, h0.y, h1.x, h1.y, h2.x, h2.y, h3.x, h3.y};
}

// Lane (n = lane % 16, kg = lane / 16) loads 16 contiguous bytes per instruction, so that the four kg lanes of a row
// fetch 64 contiguous bytes and adjacent instructions finish the cache line; v_permlane{16,32}_swap then hands every
// MFMA the 8 codes per lane it needs from ONE block:
//   Q8_0: a load covers two blocks of the row (kg 0, 1: the even one, kg 2, 3: the odd one); swapping the upper 8 bytes
//         of the lower 32 lanes with the lower 8 bytes of the upper 32 lanes leaves the even block in the first two
//         dwords of all four lanes and the odd block in the last two; lane kg then holds weights
//         16 (kg & 1) + 8 (kg >> 1) .. + 7 of its block.
//   Q4_0: a load is one whole block per lane (16 bytes of nibbles), four blocks per row; a 4 x 4 transposition of dwords
//         over the kg lanes (swap by 32 lanes, then by 16) leaves dword kg of block c in register c: weights
//         4 kg .. 4 kg + 3 (low nibbles) and 16 + 4 kg .. + 3 (high nibbles).
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));

template <int QT, bool TAIL>   // TAIL: width % 256 != 0
__global__ __launch_bounds__(256, 2) void gemm_blk_nb(const _Float16* hxhi, const _Float16* hxlo, const _Float16* hsxhi, const _Float16* hsxlo, const float* hsinvb, const int hcols, const int hntok, const int hS, const int hntiles, const NbParams p)
{
  extern __shared__ __align__(16) unsigned char nb_smem[];
  const int S = hS;
  _Float16* xs = reinterpret_cast<_Float16*>(nb_smem);              // [S][16][NB_LDX]
  float* sinv_s = reinterpret_cast<float*>(xs + S * NB_SC * NB_LDX);  // [S][8]
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: segment lookups and loop bounds stay scalar
  const int n = lane & 15, kg = lane >> 4;
  const int K = hcols, nsb = (K + 255) >> 8, nb32 = K >> 5;
  const int slice = blockIdx.y, sb0 = slice * S, nS = min(S, nsb - sb0);
  const int row_bytes = QT != CAI_Q4_0 ? K : (K >> 1);
  const int aux_row_bytes = nb32 * 2;
  const int tile0 = blockIdx.x * 4 + wave;
  const int n_it = tile0 < hntiles ? (hntiles - tile0 + p.tile_stride - 1) / p.tile_stride : 0;
  // an item = 32 rows x 128 bytes of quants: 4 blocks of Q8_0 (half a group) or 8 blocks of Q4_0 (a whole group)
  constexpr int IB = QT != CAI_Q4_0 ? 4 : 8;     // blocks per item
  constexpr int IPG = 8 / IB;                    // items per group
  const int nI = nS * IPG;                       // items per tile
  const int nq = n_it * nI;

  struct WRegs { uint32_t d[2][IB / 2]; uint4 q[2][2]; };
  auto locate = [&](int tile, const NbSeg*& sg, int& R0) {
    int sgi = 0, t0 = 0;
    if (p.n_seg > 1 && tile >= p.seg[0].tile_end) { sgi = 1; t0 = p.seg[0].tile_end; }
    if (p.n_seg > 2 && tile >= p.seg[1].tile_end) { sgi = 2; t0 = p.seg[1].tile_end; }
    sg = &p.seg[sgi]; R0 = (tile - t0) * 32;
  };
  // Loads are never conditional: past the wave's last item the last one is fetched again (a cache hit).  A load under a
  // branch would make the compiler wait for ALL outstanding loads at every join.
  auto load_w = [&](int q, WRegs& r) {
    const int qc = max(min(q, nq - 1), 0);
    const int tile = min(tile0 + (qc / nI) * p.tile_stride, hntiles - 1), it = qc % nI;
    const int g0 = (sb0 + it / IPG) * 8 + (it % IPG) * IB;                         // first block of the item
    const NbSeg* sg; int R0; locate(tile, sg, R0);
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      const int64_t row = min(R0 + 16 * hh + n, sg->rows - 1);                  // tail rows: re-read the last row
      const uint8_t* qrow = sg->w + row * row_bytes;
      const uint8_t* arow = sg->aux + row * aux_row_bytes;
      if (QT == CAI_I8ROW) { r.d[hh][0] = 0x3C003C00u; r.d[hh][IB / 2 - 1] = 0x3C003C00u; }   // per-row int8: every block scale is 1
      else if (!TAIL) {
        if (QT == CAI_Q8_0) { const uint2 t = *reinterpret_cast<const uint2*>(arow + g0 * 2); r.d[hh][0] = t.x; r.d[hh][IB / 2 - 1] = t.y; }
        else { const uint4 t = *reinterpret_cast<const uint4*>(arow + g0 * 2); r.d[hh][0] = t.x; r.d[hh][1] = t.y; r.d[hh][IB / 2 - 2] = t.z; r.d[hh][IB / 2 - 1] = t.w; }
      } else {                                                                    // the row may end inside the item: absent blocks get scale 0
#pragma unroll
        for (int i = 0; i < IB / 2; i++) {
          const int b0 = g0 + 2 * i;
          const uint32_t lo16 = *reinterpret_cast<const uint16_t*>(arow + min(b0, nb32 - 1) * 2);
          const uint32_t hi16 = *reinterpret_cast<const uint16_t*>(arow + min(b0 + 1, nb32 - 1) * 2);
          r.d[hh][i] = (b0 < nb32 ? lo16 : 0u) | ((b0 + 1 < nb32 ? hi16 : 0u) << 16);
        }
      }
#pragma unroll
      for (int j = 0; j < 2; j++) {
        int off = g0 * (QT != CAI_Q4_0 ? 32 : 16) + 64 * j + 16 * kg;
        if (TAIL) off = max(0, min(off, row_bytes - 16));                         // stays inside the row; such codes meet scale 0
        r.q[hh][j] = *reinterpret_cast<const uint4*>(qrow + off);
      }
    }
  };
  WRegs w0, w1, w2, w3;

  // ---- stage this slice of the activations: nS x 16 columns x 256 halfs (zero beyond the width), block scales ----
  // All requests of a thread are issued before the first value is stored (four at a time): one memory round trip per four
  // chunks.  Requests are unconditional (clamped token and column), what is absent is zeroed on the way to LDS.
  {
    const int n_si = nS * NB_TK;
    const int si_i = min((int)threadIdx.x, n_si - 1), si_tok = si_i % NB_TK, si_s = si_i / NB_TK;
    const float siv = hsinvb[(int64_t)min(si_tok, hntok - 1) * nsb + sb0 + si_s];
    const int total = nS * NB_SC * 32;
    for (int base = 0; base < total; base += 4 * 256) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int idx = min(base + u * 256 + (int)threadIdx.x, total - 1);
        const int chunk = idx & 31, col = (idx >> 5) % NB_SC, s = (idx >> 5) / NB_SC, tok = min(col % NB_TK, hntok - 1);
        int k = (sb0 + s) * 256 + chunk * 8;
        if (TAIL) k = min(k, K - 8);
        v[u] = *reinterpret_cast<const uint4*>(((col / NB_TK) ? hxlo : hxhi) + (int64_t)tok * K + k);
      }
      if (base == 0) { load_w(0, w0); load_w(1, w1); load_w(2, w2); load_w(3, w3); }   // (behind the first activation requests: see gemm_q4k_nb)
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int idx = base + u * 256 + (int)threadIdx.x;
        if (idx < total) {
          const int chunk = idx & 31, col = (idx >> 5) % NB_SC, s = (idx >> 5) / NB_SC;
          const bool present = (col % NB_TK) < hntok && (!TAIL || (sb0 + s) * 256 + chunk * 8 < K);
          *reinterpret_cast<uint4*>(xs + (s * NB_SC + col) * NB_LDX + chunk * 8) = present ? v[u] : make_uint4(0, 0, 0, 0);
        }
      }
    }
    if ((int)threadIdx.x < n_si) sinv_s[si_i] = si_tok < hntok ? siv : 0.0f;
  }
  __syncthreads();

  float acc[2][4], g[2][4];
  const int xoff = QT != CAI_Q4_0 ? 16 * (kg & 1) + 8 * (kg >> 1) : 4 * kg;   // this lane's first weight within a block
  auto compute = [&](const WRegs& r, int q) {
    const int it = q % nI, s = it / IPG, part = it % IPG;
    if (it == 0) {
#pragma unroll
      for (int hh = 0; hh < 2; hh++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[hh][i] = 0.0f;
    }
    if (part == 0) {
#pragma unroll
      for (int hh = 0; hh < 2; hh++)
#pragma unroll
        for (int i = 0; i < 4; i++) g[hh][i] = 0.0f;
    }
    const _Float16* xcol = xs + (s * NB_SC + n) * NB_LDX + part * IB * 32 + xoff;
    const float4_t z4 = {0.0f, 0.0f, 0.0f, 0.0f};
    auto block = [&](int hh, int b, uint32_t c0, uint32_t c1) {
      half8_t X;
      if (QT != CAI_Q4_0) X = *reinterpret_cast<const half8_t*>(xcol + 32 * b);
      else {
        const half4_t x0 = *reinterpret_cast<const half4_t*>(xcol + 32 * b);
        const half4_t x1 = *reinterpret_cast<const half4_t*>(xcol + 32 * b + 16);
        X = half8_t{x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
      }
      const half8_t W = codes_to_half8<QT>(c0, c1);
      const float4_t C = __builtin_amdgcn_mfma_f32_16x16x32_f16(X, W, z4, 0, 0, 0);
      const uint32_t dw = r.d[hh][b >> 1];
      const float d = __half2float(__ushort_as_half((unsigned short)((b & 1) ? (dw >> 16) : (dw & 0xffffu))));
#pragma unroll
      for (int i = 0; i < 4; i++) g[hh][i] = fmaf(d, C[i], g[hh][i]);
    };
#pragma unroll
    for (int j = 0; j < 2; j++) {
#pragma unroll
      for (int hh = 0; hh < 2; hh++) {
        const uint4 v = r.q[hh][j];
        if (QT != CAI_Q4_0) {
          const uint2_t s0 = __builtin_amdgcn_permlane32_swap(v.x, v.z, false, false);   // .x: even block, .y: odd block
          const uint2_t s1 = __builtin_amdgcn_permlane32_swap(v.y, v.w, false, false);
          block(hh, 2 * j, s0.x, s1.x);
          block(hh, 2 * j + 1, s0.y, s1.y);
        } else {
          const uint2_t t02 = __builtin_amdgcn_permlane32_swap(v.x, v.z, false, false);
          const uint2_t t13 = __builtin_amdgcn_permlane32_swap(v.y, v.w, false, false);
          const uint2_t u01 = __builtin_amdgcn_permlane16_swap(t02.x, t13.x, false, false);  // blocks 4 j, 4 j + 1
          const uint2_t u23 = __builtin_amdgcn_permlane16_swap(t02.y, t13.y, false, false);  // blocks 4 j + 2, 4 j + 3
          block(hh, 4 * j, u01.x, 0u); block(hh, 4 * j + 1, u01.y, 0u);
          block(hh, 4 * j + 2, u23.x, 0u); block(hh, 4 * j + 3, u23.y, 0u);
        }
      }
    }
    if (part != IPG - 1) return;
    // result row 4 kg + i of the tile = token (4 kg + i) % 8, its hi (kg < 2) or lo (kg >= 2) part
    const float4 si = *reinterpret_cast<const float4*>(&sinv_s[s * NB_TK + 4 * (kg & 1)]);
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      acc[hh][0] = fmaf(si.x, g[hh][0], acc[hh][0]); acc[hh][1] = fmaf(si.y, g[hh][1], acc[hh][1]);
      acc[hh][2] = fmaf(si.z, g[hh][2], acc[hh][2]); acc[hh][3] = fmaf(si.w, g[hh][3], acc[hh][3]);
    }
    if (it != nI - 1) return;
    // ---- the slice's contribution of this tile: hi + lo parts meet across kg ^ 2; lanes kg < 2 store four tokens ----
    const int tile = tile0 + (q / nI) * p.tile_stride;
    const NbSeg* sg; int R0; locate(tile, sg, R0);
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      const int row = R0 + 16 * hh + n;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float tot = acc[hh][i] + __shfl_xor(acc[hh][i], 32, 64);
        const int tok = 4 * kg + i;
        if (kg < 2 && tok < hntok && row < sg->rows)
          p.part[((int64_t)slice * hntok + tok) * p.part_stride + sg->y_off + row] = tot;
      }
    }
  };

  // ring of four items: three are in flight while one is consumed
  for (int q = 0; q < nq; q += 4) {
    compute(w0, q); load_w(q + 4, w0);
    if (q + 1 < nq) compute(w1, q + 1);
    load_w(q + 5, w1);
    if (q + 2 < nq) compute(w2, q + 2);
    load_w(q + 6, w2);
    if (q + 3 < nq) compute(w3, q + 3);
    load_w(q + 7, w3);
  }
}

// ------------------------------------------------------------------------------------------
// Q6_K (256-weight super-blocks of 210 bytes: 128 of low nibbles, 64 of 2-bit high parts, 16 signed scales, one f16;
// neural/neuralgguf.pas:639-717).  Scales belong to 16 weights of a ROW, so the operands are swapped as for the 32-weight
// block types and one v_mfma_f32_16x16x16_f16 covers exactly one scale group: the lane (weight row lane % 16, kg) supplies
// the codes 4 kg .. 4 kg + 3 of the group (q - 32, exact in f16) and multiplies the four results by d * scale, both values
// it loaded itself.  Group g = 8 nh + 2 j + h of a super-block lies in bytes 16 (4 nh + 2 (j & 1) + h) .. + 15 of ql
// (nibble j >> 1) and bytes 16 (2 nh + h) .. + 15 of qh (2-bit field j).  Lane kg loads the 16-byte chunks kg and kg + 4
// of ql and chunk kg of qh, and a 4 x 4 transposition of dwords over the kg lanes leaves dword kg of chunk c in register
// c.  Resident form: 192-byte ql | qh records, a plane of scales and a plane of d (the file's 210-byte blocks are only
// 2-byte aligned, and unaligned requests stream at two thirds of the rate).
// ------------------------------------------------------------------------------------------
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// NT groups of 8 tokens share every converted weight operand and scale: 9..16 tokens take one pass with NT = 2.
template <int NT>
__global__ __launch_bounds__(256, 2) void gemm_q6k_nb(const _Float16* hxhi, const _Float16* hxlo, const _Float16* hsxhi, const _Float16* hsxlo, const float* hsinvb, const int hcols, const int hntok, const int hS, const int hntiles, const NbParams p)
{
  extern __shared__ __align__(16) unsigned char nb_smem[];
  const int S = hS;
  constexpr int NC = NT * NB_SC, NTOK = NT * NB_TK;                 // staged columns per super-block: group t holds tokens 8t..8t+7 as 8 hi + 8 lo
  _Float16* xs = reinterpret_cast<_Float16*>(nb_smem);              // [S][NC][NB_LDX]
  float* sinv_s = reinterpret_cast<float*>(xs + S * NC * NB_LDX);    // [S][NTOK]
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 15, kg = lane >> 4;
  const int K = hcols, nsb = K >> 8;
  const int slice = blockIdx.y, sb0 = slice * S, nS = min(S, nsb - sb0);
  const int tile0 = blockIdx.x * 4 + wave;
  const int n_it = tile0 < hntiles ? (hntiles - tile0 + p.tile_stride - 1) / p.tile_stride : 0;
  const int nq = n_it * nS;                      // (tile, super-block) items of this wave

  struct WRegs { u32x4_t ql[2][2], qh[2], sc[2]; uint32_t d[2]; };
  auto locate = [&](int tile, const NbSeg*& sg, int& R0) {
    int sgi = 0, t0 = 0;
    if (p.n_seg > 1 && tile >= p.seg[0].tile_end) { sgi = 1; t0 = p.seg[0].tile_end; }
    if (p.n_seg > 2 && tile >= p.seg[1].tile_end) { sgi = 2; t0 = p.seg[1].tile_end; }
    sg = &p.seg[sgi]; R0 = (tile - t0) * 32;
  };
  // unconditional, clamped: past the wave's last item the last one is fetched again (a cache hit)
  auto load_w = [&](int q, WRegs& r) {
    const int qc = max(min(q, nq - 1), 0);
    const int tile = min(tile0 + (qc / nS) * p.tile_stride, hntiles - 1), sb = sb0 + qc % nS;
    const NbSeg* sg; int R0; locate(tile, sg, R0);
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      const int64_t b = (int64_t)min(R0 + 16 * hh + n, sg->rows - 1) * nsb + sb;   // tail rows: re-read the last row
      const uint8_t* blk = sg->w + b * 192;
      r.ql[hh][0] = *reinterpret_cast<const u32x4_t*>(blk + 16 * kg);
      r.ql[hh][1] = *reinterpret_cast<const u32x4_t*>(blk + 64 + 16 * kg);
      r.qh[hh] = *reinterpret_cast<const u32x4_t*>(blk + 128 + 16 * kg);
      r.sc[hh] = *reinterpret_cast<const u32x4_t*>(sg->aux + b * 16);
      r.d[hh] = *reinterpret_cast<const uint16_t*>(sg->aux2 + b * 2);
    }
  };
  WRegs wa, wb, wc;

  // ---- stage this slice of the activations: nS x 16 columns x 256 halfs, block scales (four requests per turn) ----
  {
    const int n_si = nS * NTOK;
    const int total = nS * NC * 32;
    for (int base = 0; base < total; base += 4 * 256) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int idx = min(base + u * 256 + (int)threadIdx.x, total - 1);
        const int chunk = idx & 31, col = (idx >> 5) % NC, s = (idx >> 5) / NC;
        const int tok = min((col / NB_SC) * NB_TK + col % NB_TK, hntok - 1);
        v[u] = *reinterpret_cast<const uint4*>((((col % NB_SC) / NB_TK) ? hxlo : hxhi) + (int64_t)tok * K + (sb0 + s) * 256 + chunk * 8);
      }
      if (base == 0) { load_w(0, wa); load_w(1, wb); }   // (behind the first activation requests: see gemm_q4k_nb)
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int idx = base + u * 256 + (int)threadIdx.x;
        if (idx < total) {
          const int chunk = idx & 31, col = (idx >> 5) % NC, s = (idx >> 5) / NC;
          const int tok = (col / NB_SC) * NB_TK + col % NB_TK;
          *reinterpret_cast<uint4*>(xs + (s * NC + col) * NB_LDX + chunk * 8) = tok < hntok ? v[u] : make_uint4(0, 0, 0, 0);
        }
      }
    }
    for (int i = threadIdx.x; i < n_si; i += 256) {
      const int tok = i % NTOK, s = i / NTOK;
      sinv_s[i] = tok < hntok ? hsinvb[(int64_t)tok * nsb + sb0 + s] : 0.0f;
    }
  }
  __syncthreads();

  float acc[NT][2][4];
  auto compute = [&](const WRegs& r, int q) {
    const int s = q % nS;
    if (s == 0) {
#pragma unroll
      for (int t = 0; t < NT; t++)
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
          for (int i = 0; i < 4; i++) acc[t][hh][i] = 0.0f;
    }
    const _Float16* xcol = xs + (s * NC + n) * NB_LDX + 4 * kg;
    const float4_t z4 = {0.0f, 0.0f, 0.0f, 0.0f};
    const half2_t o2 = {(_Float16)(-1056.0f), (_Float16)(-1056.0f)};   // 1024 + q - 1056 = q - 32
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      float g[NT][4];
#pragma unroll
      for (int t = 0; t < NT; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) g[t][i] = 0.0f;
      // dword kg of every chunk: ql chunks 0..7 in lq[0..7], qh chunks 0..3 in hq[0..3]
      uint32_t lq[8], hq[4];
#pragma unroll
      for (int a = 0; a < 3; a++) {
        const u32x4_t v = a < 2 ? r.ql[hh][a] : r.qh[hh];
        const uint2_t t02 = __builtin_amdgcn_permlane32_swap(v.x, v.z, false, false);
        const uint2_t t13 = __builtin_amdgcn_permlane32_swap(v.y, v.w, false, false);
        const uint2_t u01 = __builtin_amdgcn_permlane16_swap(t02.x, t13.x, false, false);
        const uint2_t u23 = __builtin_amdgcn_permlane16_swap(t02.y, t13.y, false, false);
        uint32_t* dst = a < 2 ? lq + 4 * a : hq;
        dst[0] = u01.x; dst[1] = u01.y; dst[2] = u23.x; dst[3] = u23.y;
      }
      const float d = __half2float(__ushort_as_half((unsigned short)r.d[hh]));
      const uint32_t scw[4] = {r.sc[hh].x, r.sc[hh].y, r.sc[hh].z, r.sc[hh].w};
#pragma unroll
      for (int gi = 0; gi < 16; gi++) {
        const int nh = gi >> 3, j = (gi >> 1) & 3, h = gi & 1;
        const uint32_t lo = (lq[4 * nh + 2 * (j & 1) + h] >> (4 * (j >> 1))) & 0x0f0f0f0fu;
        const uint32_t hf = hq[2 * nh + h];
        const uint32_t hi = (j == 0 ? (hf << 4) : j == 1 ? (hf << 2) : j == 2 ? hf : (hf >> 2)) & 0x30303030u;
        const uint32_t c = lo | hi;
        const half2_t w01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, c, 0x04010400u)) + o2;
        const half2_t w23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, c, 0x04030402u)) + o2;
        const half4_t W = {w01.x, w01.y, w23.x, w23.y};
        const float ds = d * (float)(int)(int8_t)((scw[gi >> 2] >> (8 * (gi & 3))) & 0xffu);
#pragma unroll
        for (int t = 0; t < NT; t++) {
          const half4_t X = *reinterpret_cast<const half4_t*>(xcol + t * NB_SC * NB_LDX + 16 * gi);
          const float4_t C = __builtin_amdgcn_mfma_f32_16x16x16f16(X, W, z4, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 4; i++) g[t][i] = fmaf(ds, C[i], g[t][i]);
        }
      }
      // result row 4 kg + i of a group = token (4 kg + i) % 8 of the group, its hi (kg < 2) or lo (kg >= 2) part
#pragma unroll
      for (int t = 0; t < NT; t++) {
        const float4 si = *reinterpret_cast<const float4*>(&sinv_s[s * NTOK + t * NB_TK + 4 * (kg & 1)]);
        acc[t][hh][0] = fmaf(si.x, g[t][0], acc[t][hh][0]); acc[t][hh][1] = fmaf(si.y, g[t][1], acc[t][hh][1]);
        acc[t][hh][2] = fmaf(si.z, g[t][2], acc[t][hh][2]); acc[t][hh][3] = fmaf(si.w, g[t][3], acc[t][hh][3]);
      }
    }
    if (s != nS - 1) return;
    // ---- the slice's contribution of this tile: hi + lo parts meet across kg ^ 2; lanes kg < 2 store four tokens ----
    const int tile = tile0 + (q / nS) * p.tile_stride;
    const NbSeg* sg; int R0; locate(tile, sg, R0);
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
      for (int hh = 0; hh < 2; hh++) {
        const int row = R0 + 16 * hh + n;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const float tot = acc[t][hh][i] + __shfl_xor(acc[t][hh][i], 32, 64);
          const int tok = t * NB_TK + 4 * kg + i;
          if (kg < 2 && tok < hntok && row < sg->rows)
            p.part[((int64_t)slice * hntok + tok) * p.part_stride + sg->y_off + row] = tot;
        }
      }
  };

  for (int q = 0; q < nq; q += 3) {
    load_w(q + 2, wc); compute(wa, q);
    load_w(q + 3, wa); if (q + 1 < nq) compute(wb, q + 1);
    load_w(q + 4, wb); if (q + 2 < nq) compute(wc, q + 2);
  }
}

// ------------------------------------------------------------------------------------------
// Activation pre-pass: one work-group per (256-block, token).  Source of the block:
//   SRC 0  x[t][k]                                                       (a plain activation row)
//   SRC 1  res[t][k] + bias[k] + sum_s part[s][t][k], written back to res (a projection added to the residual stream)
//   SRC 2  u * silu(g), u = inv_t * sum_s part[s][t][k] + bias[k], g likewise at column half + k   (SwiGLU of a product)
// then v = gain[k] * value (gain optional), per-block power-of-two scale, hi/lo halfs, sub-block sums, and the block's
// sum of squares of the un-gained value (for the RMSNorm the consumer of the product applies).
// ------------------------------------------------------------------------------------------
struct NbPrepParams {
  const float* x; int64_t x_stride;             // SRC 0
  float* res; int64_t res_stride;               // SRC 1 (in/out)
  const float* part; int64_t part_stride; int n_slices; int n_tok;   // SRC 1, 2
  const float* bias;                            // SRC 1: [K]; SRC 2: [2*half]
  int half;                                     // SRC 2: column of the gate partner
  const float* in_ssq; int in_nsb; int in_K; float in_eps;   // SRC 2: RMSNorm of the product's input (in_ssq null = none)
  const float* gain;                            // optional, [K]
  int K;
  _Float16* hi; _Float16* lo; _Float16* sxhi; _Float16* sxlo; float* sinvb; float* ssq;
};

// Sums n values `stride` apart in index order; the requests go out eight at a time (the additions stay sequential, so the
// result does not depend on the batching).
__device__ __forceinline__ float nb_sum_strided(const float* p, int n, int64_t stride, float acc)
{
  int i = 0;
  for (; i + 8 <= n; i += 8) {
    float t[8];
#pragma unroll
    for (int u = 0; u < 8; u++) t[u] = p[(int64_t)(i + u) * stride];
#pragma unroll
    for (int u = 0; u < 8; u++) acc += t[u];
  }
  for (; i < n; i++) acc += p[(int64_t)i * stride];
  return acc;
}

__device__ __forceinline__ float nb_inv_rms(const float* ssq, int nsb, int K, float eps, int tok)
{
  const float t = nb_sum_strided(ssq + (int64_t)tok * nsb, nsb, 1, 0.0f);   // fixed order
  return 1.0f / sqrtf(t / (float)K + eps);
}

// (what the first requests need travels as leading scalar arguments, preloaded in scalar registers: hsrc = x (SRC 0) or res (SRC 1))
template <int SRC>
__global__ __launch_bounds__(256) void nb_prep_kernel(const float* hsrc, const long long hstride, const float* hpart, const long long hpstride, const float* hbias,
                                                      const float* hgain, const int hns, const int hntok, const NbPrepParams p)
{
  const int sb = blockIdx.x, tok = blockIdx.y, k = sb * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nsb = (p.K + 255) >> 8;
  const bool in = k < p.K;                       // the last block of a width that is not a multiple of 256 is short
  float v = 0.0f;
  if (!in) {}
  else if (SRC == 0) v = hsrc[(int64_t)tok * hstride + k];
  else if (SRC == 1) {
    v = hsrc[(int64_t)tok * hstride + k];
    if (hbias) v += hbias[k];
    v = nb_sum_strided(hpart + (int64_t)tok * hpstride + k, hns, (int64_t)hntok * hpstride, v);
    p.res[(int64_t)tok * p.res_stride + k] = v;
  } else {
    const float* col = hpart + (int64_t)tok * hpstride + k;
    const float up0 = nb_sum_strided(col, hns, (int64_t)hntok * hpstride, 0.0f);
    const float gate0 = nb_sum_strided(col + p.half, hns, (int64_t)hntok * hpstride, 0.0f);
    float up = up0, gate = gate0;
    if (p.in_ssq) { const float inv = nb_inv_rms(p.in_ssq, p.in_nsb, p.in_K, p.in_eps, tok); up *= inv; gate *= inv; }
    if (hbias) { up += hbias[k]; gate += hbias[p.half + k]; }
    v = silu_mul(up, gate);
  }
  const float raw = v;
  if (in && hgain) v *= hgain[k];
  __shared__ float red[8];
  float amax = fabsf(v), ss = raw * raw;
  for (int off = 32; off > 0; off >>= 1) { amax = fmaxf(amax, __shfl_xor(amax, off, 64)); ss += __shfl_xor(ss, off, 64); }
  if (lane == 0) { red[wave] = amax; red[4 + wave] = ss; }
  __syncthreads();
  const float a = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  int e = 0;
  if (a > 0.0f && a < 3.0e38f) { int ex; frexpf(a, &ex); e = 14 - ex; }   // a * 2^e in [2^13, 2^14)
  e = max(-60, min(60, e));
  const float s = ldexpf(1.0f, e);
  const float vs = v * s;
  _Float16 h, l; split_f16(vs, h, l);
  const int64_t o = (int64_t)tok * p.K + k;
  if (in) { p.hi[o] = h; p.lo[o] = l; }
  float sum = vs;
  for (int off = 16; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);   // 32-lane groups = the 8 sub-blocks
  if ((threadIdx.x & 31) == 0 && in) {
    const float q = sum * 0.03125f;
    _Float16 sh, sl; split_f16(q, sh, sl);
    const int64_t b = (int64_t)tok * (p.K >> 5) + sb * 8 + (threadIdx.x >> 5);
    p.sxhi[b] = sh; p.sxlo[b] = sl;
  }
  if (threadIdx.x == 0) {
    p.sinvb[(int64_t)tok * nsb + sb] = ldexpf(1.0f, -e);
    p.ssq[(int64_t)tok * nsb + sb] = (red[4] + red[5]) + (red[6] + red[7]);
  }
}

// y[t][y_off + r] = inv_t * sum_s part[s][t][y_off + r] + bias[r] (+ residual): the plain consumer of a product
struct NbReduceParams {
  NbSeg seg[3]; int n_seg;
  const float* part; int64_t part_stride; int n_slices; int n_tok;
  const float* in_ssq; int in_nsb; int in_K; float in_eps;
  float* y; int64_t y_stride; const float* residual;
  int width;                                    // columns covered (sum of the segments)
};
__global__ __launch_bounds__(256) void nb_reduce_kernel(const float* hpart, const long long hpstride, const int hns, const int hntok, const int hwidth, const NbReduceParams p)
{
  const int tok = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= hwidth) return;
  int sgi = 0;
  if (p.n_seg > 1 && c >= p.seg[1].y_off) sgi = 1;
  if (p.n_seg > 2 && c >= p.seg[2].y_off) sgi = 2;
  float v = nb_sum_strided(hpart + (int64_t)tok * hpstride + c, hns, (int64_t)hntok * hpstride, 0.0f);
  if (p.in_ssq) v *= nb_inv_rms(p.in_ssq, p.in_nsb, p.in_K, p.in_eps, tok);
  if (p.seg[sgi].row_scale) v *= p.seg[sgi].row_scale[c - p.seg[sgi].y_off];   // per-row int8: (sum code * x) * scale, then bias
  if (p.seg[sgi].bias) v += p.seg[sgi].bias[c - p.seg[sgi].y_off];
  const int64_t o = (int64_t)tok * p.y_stride + c;
  if (p.residual) v += p.residual[o];
  p.y[o] = v;
}

// ------------------------------------------------------------------------------------------
// host side: workspace + the record of the product in flight (one stream, calls are sequential)
// ------------------------------------------------------------------------------------------
namespace {
struct NbWs {
  _Float16 *hi = nullptr, *lo = nullptr, *sxhi = nullptr, *sxlo = nullptr; float *sinvb = nullptr, *ssq[2] = {nullptr, nullptr}, *part = nullptr;
  size_t cap_k = 0, cap_part = 0;
  int generation = 0;
  int cur = 0;                // ssq buffer the last pre-pass wrote
};
NbWs g_nb;
struct NbProduct {            // what the last nb_gemm left in `part`
  NbSeg seg[3]; int n_seg = 0; int n_slices = 0; int n_tok = 0; int64_t part_stride = 0; int width = 0;
  const float* in_ssq = nullptr; int in_nsb = 0, in_K = 0; float in_eps = 0.0f;
};
NbProduct g_prod;
const float* g_pending_ssq = nullptr; int g_pending_K = 0; float g_pending_eps = 0.0f;   // norm of the activations in the planes
}  // namespace

int nb_ws_generation() { return g_nb.generation; }

// cai_shutdown: the workspace goes back to the device; decoders that captured graphs against it see a new generation
void nb_release()
{
  void* q[] = {g_nb.hi, g_nb.lo, g_nb.sxhi, g_nb.sxlo, g_nb.sinvb, g_nb.ssq[0], g_nb.ssq[1], g_nb.part};
  for (void* v : q) if (v) (void)hipFree(v);
  const int gen = g_nb.generation + 1;
  g_nb = NbWs(); g_nb.generation = gen;
  g_prod = NbProduct(); g_pending_ssq = nullptr; g_pending_K = 0;
}

// Reserves planes for k_max columns and a partial buffer of part_floats floats (never inside a stream capture).
int nb_reserve(int k_max, size_t part_floats)
{
  const size_t need_k = (size_t)NB_TMAX * k_max;
  if (need_k > g_nb.cap_k) {
    CAI_HIP(hipStreamSynchronize(ctx().stream));
    void* old[] = {g_nb.hi, g_nb.lo, g_nb.sxhi, g_nb.sxlo, g_nb.sinvb, g_nb.ssq[0], g_nb.ssq[1]};
    for (void* q : old) if (q) (void)hipFree(q);
    CAI_HIP(hipMalloc((void**)&g_nb.hi, need_k * 2)); CAI_HIP(hipMalloc((void**)&g_nb.lo, need_k * 2));
    CAI_HIP(hipMalloc((void**)&g_nb.sxhi, need_k / 32 * 2 + 64)); CAI_HIP(hipMalloc((void**)&g_nb.sxlo, need_k / 32 * 2 + 64));
    const size_t nblk = (size_t)NB_TMAX * ((k_max + 255) / 256);
    CAI_HIP(hipMalloc((void**)&g_nb.sinvb, nblk * 4 + 64));
    CAI_HIP(hipMalloc((void**)&g_nb.ssq[0], nblk * 4 + 64)); CAI_HIP(hipMalloc((void**)&g_nb.ssq[1], nblk * 4 + 64));
    g_nb.cap_k = need_k; g_nb.generation++;
  }
  if (part_floats > g_nb.cap_part) {
    CAI_HIP(hipStreamSynchronize(ctx().stream));
    if (g_nb.part) (void)hipFree(g_nb.part);
    CAI_HIP(hipMalloc((void**)&g_nb.part, part_floats * 4));
    g_nb.cap_part = part_floats; g_nb.generation++;
  }
  return CAI_OK;
}

// How a product over `cols` columns and `tiles` 32-row tiles is cut: S super-blocks per K slice and gx row groups, so
// that gx * slices work-groups fit the chip in ONE round (three work-groups share a CU) and the waves' shares come out
// even.  A wave's share is ceil(tiles / (4 gx)) tiles of S items each (item = 32 rows x one super-block) plus the
// partial result every (tile, slice) writes and its consumer re-reads, priced at 0.45 item.
static void nb_geometry(int cols, int tiles, int& S, int& n_slices, int& gx, int& tile_stride, int s_max = NB_SMAX)
{
  const int nsb = (cols + 255) >> 8, slots = 3 * ctx().n_cu;
  const int s_lo = std::min(2, nsb), s_hi = std::min(s_max, nsb);
  float best = 3.0e38f;
  S = s_lo;
  for (int s = s_lo; s <= s_hi; s++) {
    const int ns = (nsb + s - 1) / s;
    const int g = std::max(1, std::min((tiles + 3) / 4, slots / ns));
    const int share = (tiles + 4 * g - 1) / (4 * g);
    const float cost = (float)share * ((float)s + 0.45f);
    if (cost < best) { best = cost; S = s; gx = g; n_slices = ns; }
  }
  tile_stride = gx * 4;
}
// upper bound of the slice count for a width (sizes the partial buffer): S never drops below min(2, blocks per row)
int nb_max_slices(int cols) { const int nsb = std::max((cols + 255) >> 8, 1); const int s = std::min(2, nsb); return (nsb + s - 1) / s; }

static int nb_prep_launch(int src, NbPrepParams& p, int n_tok)
{
  if (p.K % 32) return set_error(CAI_ERR_UNSUPPORTED, "small-batch pre-pass: width %d is not a multiple of 32", p.K);
  if ((size_t)NB_TMAX * p.K > g_nb.cap_k || n_tok > NB_TMAX) return set_error(CAI_ERR_STATE, "small-batch pre-pass: workspace not reserved for %d x %d", n_tok, p.K);
  g_nb.cur ^= 1;
  p.hi = g_nb.hi; p.lo = g_nb.lo; p.sxhi = g_nb.sxhi; p.sxlo = g_nb.sxlo; p.sinvb = g_nb.sinvb; p.ssq = g_nb.ssq[g_nb.cur];
  const dim3 grid((p.K + 255) >> 8, n_tok);
  const float* hsrc = src == 0 ? p.x : src == 1 ? p.res : nullptr;
  const long long hstride = src == 0 ? p.x_stride : p.res_stride, hps = p.part_stride;
  if (src == 0) hipLaunchKernelGGL(nb_prep_kernel<0>, grid, dim3(256), 0, ctx().stream, hsrc, hstride, p.part, hps, p.bias, p.gain, p.n_slices, p.n_tok, p);
  else if (src == 1) hipLaunchKernelGGL(nb_prep_kernel<1>, grid, dim3(256), 0, ctx().stream, hsrc, hstride, p.part, hps, p.bias, p.gain, p.n_slices, p.n_tok, p);
  else hipLaunchKernelGGL(nb_prep_kernel<2>, grid, dim3(256), 0, ctx().stream, hsrc, hstride, p.part, hps, p.bias, p.gain, p.n_slices, p.n_tok, p);
  return CAI_OK;
}
static void nb_set_pending_norm(const float* gain, int K, float eps)
{
  g_pending_ssq = gain ? g_nb.ssq[g_nb.cur] : nullptr; g_pending_K = K; g_pending_eps = eps;
}

// planes <- x (RMSNorm with `gain` is completed by the consumer of the next product)
int nb_prep_plain(const float* x, int64_t x_stride, const float* gain, float eps, int K, int n_tok)
{
  NbPrepParams p{}; p.x = x; p.x_stride = x_stride; p.gain = gain; p.K = K;
  const int rc = nb_prep_launch(0, p, n_tok); if (rc) return rc;
  nb_set_pending_norm(gain, K, eps);
  return CAI_OK;
}
// res <- res + last product (+bias); planes <- res (norm as above).  The product must not itself carry a pending norm.
int nb_prep_residual(float* res, int64_t res_stride, const float* gain, float eps, int K, int n_tok)
{
  if (g_prod.n_seg != 1 || g_prod.width != K || g_prod.n_tok != n_tok || g_prod.in_ssq || g_prod.seg[0].row_scale)
    return set_error(CAI_ERR_STATE, "small-batch residual pre-pass: no matching product in flight");
  NbPrepParams p{}; p.res = res; p.res_stride = res_stride; p.part = g_nb.part; p.part_stride = g_prod.part_stride; p.n_slices = g_prod.n_slices; p.n_tok = n_tok;
  p.bias = g_prod.seg[0].bias; p.gain = gain; p.K = K;
  const int rc = nb_prep_launch(1, p, n_tok); if (rc) return rc;
  nb_set_pending_norm(gain, K, eps);
  g_prod.n_seg = 0;
  return CAI_OK;
}
// planes <- SwiGLU of the last product (rows [0, half) up, [half, 2 half) gate)
int nb_prep_swiglu(int half, int n_tok)
{
  if (g_prod.n_seg != 1 || g_prod.width != 2 * half || g_prod.n_tok != n_tok || g_prod.seg[0].row_scale) return set_error(CAI_ERR_STATE, "small-batch SwiGLU pre-pass: no matching product in flight");
  NbPrepParams p{}; p.part = g_nb.part; p.part_stride = g_prod.part_stride; p.n_slices = g_prod.n_slices; p.n_tok = n_tok;
  p.bias = g_prod.seg[0].bias; p.half = half; p.in_ssq = g_prod.in_ssq; p.in_nsb = g_prod.in_nsb; p.in_K = g_prod.in_K; p.in_eps = g_prod.in_eps; p.K = half;
  const int rc = nb_prep_launch(2, p, n_tok); if (rc) return rc;
  nb_set_pending_norm(nullptr, half, 0.0f);
  g_prod.n_seg = 0;
  return CAI_OK;
}

// Weight types with a small-batch kernel.  Q4_K super-blocks make the width a multiple of 256 by construction.
bool nb_supported(const cai_qw_s* w)
{
  if (w->qtype == CAI_Q4_K || w->qtype == CAI_Q5_K || w->qtype == CAI_Q6_K) return w->cols % 256 == 0 && w->cols >= 256;
  return (w->qtype == CAI_Q8_0 || w->qtype == CAI_Q4_0 || w->qtype == CAI_I8ROW) && w->cols % 32 == 0 && w->cols >= 32;   // per-row int8: unit block scales, the row scale is applied by nb_reduce
}

// (the activation planes, the width and the slice geometry travel as leading scalar arguments: they arrive preloaded in scalar
//  registers, so the first requests do not wait for a round trip to the argument block; see the Makefile)
template <void (*Kernel)(const _Float16*, const _Float16*, const _Float16*, const _Float16*, const float*, int, int, int, int, const NbParams)>
static void nb_launch(const NbParams& p, int gx, int n_slices, size_t lds)
{
  static bool attr_done = false;   // one flag per kernel
  if (!attr_done) { (void)hipFuncSetAttribute((const void*)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); attr_done = true; }
  hipLaunchKernelGGL(Kernel, dim3(gx, n_slices), dim3(256), lds, ctx().stream, p.xhi, p.xlo, p.sxhi, p.sxlo, p.sinvb, p.cols, p.n_tok, p.sb_per_slice, p.n_tiles, p);
}

int nb_pass_tokens(const cai_qw_s* w);

// partials <- [W0; W1; W2] . planes.  The matrices share the width; those of one type share a launch (a Q4_K_M file keeps
// attn_v of some blocks in Q6_K beside Q4_K attn_q and attn_k), and every launch cuts the columns into the same slices.
int nb_gemm(const cai_qw_s* const* ws, const int* y_off, int n_w, int n_tok)
{
  if (n_w < 1 || n_w > 3 || n_tok < 1 || n_tok > nb_pass_tokens(ws[0])) return set_error(CAI_ERR_UNSUPPORTED, "small-batch gemm: %d matrices, %d tokens", n_w, n_tok);
  NbParams base{};
  base.cols = (int)ws[0]->cols;
  NbSeg segs[3];
  int tiles = 0, width = 0;
  for (int i = 0; i < n_w; i++) {
    if (!nb_supported(ws[i]) || ws[i]->cols != ws[0]->cols || n_tok > nb_pass_tokens(ws[i]))
      return set_error(CAI_ERR_UNSUPPORTED, "small-batch gemm: matrix %d type %d width %lld, %d tokens", i, ws[i]->qtype, (long long)ws[i]->cols, n_tok);
    if (i > 0 && y_off[i] < y_off[i - 1]) return set_error(CAI_ERR_INVALID, "small-batch gemm: output offsets must ascend");
    tiles += (int)((ws[i]->rows + 31) / 32);
    segs[i] = NbSeg{ws[i]->data, ws[i]->aux, qw_aux2(ws[i]), ws[i]->bias, ws[i]->qtype == CAI_I8ROW ? reinterpret_cast<const float*>(ws[i]->aux) : nullptr, (int)ws[i]->rows, y_off[i], 0};
    width = std::max(width, y_off[i] + (int)ws[i]->rows);
  }
  int S, n_slices, gx, tile_stride;
  nb_geometry(base.cols, tiles, S, n_slices, gx, tile_stride, n_tok > NB_TK ? 2 : NB_SMAX);
  const int64_t stride = (width + 3) / 4 * 4;
  if ((size_t)NB_TMAX * base.cols > g_nb.cap_k || (size_t)n_slices * n_tok * stride > g_nb.cap_part)
    return set_error(CAI_ERR_STATE, "small-batch gemm: workspace not reserved (%d slices x %d tokens x %lld)", n_slices, n_tok, (long long)stride);
  base.xhi = g_nb.hi; base.xlo = g_nb.lo; base.sxhi = g_nb.sxhi; base.sxlo = g_nb.sxlo; base.sinvb = g_nb.sinvb; base.n_tok = n_tok;
  base.part = g_nb.part; base.part_stride = stride; base.sb_per_slice = S;
  bool done[3] = {false, false, false};
  for (int i0 = 0; i0 < n_w; i0++) {
    if (done[i0]) continue;
    const int qt = ws[i0]->qtype;
    NbParams p = base;
    int sub = 0;
    for (int i = i0; i < n_w; i++) {
      if (ws[i]->qtype != qt) continue;
      done[i] = true;
      sub += (segs[i].rows + 31) / 32;
      p.seg[p.n_seg] = segs[i]; p.seg[p.n_seg].tile_end = sub; p.n_seg++;
    }
    p.n_tiles = sub;
    const int gxs = std::max(1, std::min(gx, (sub + 3) / 4));
    p.tile_stride = gxs * 4;
    if (qt == CAI_Q4_K || qt == CAI_Q5_K) {
      const size_t lds = (size_t)S * NB_SC * (NB_LDX + 8) * 2 + (size_t)S * NB_TK * 4 + 4 * 2 * 32 * 4;
      if (qt == CAI_Q4_K) nb_launch<gemm_q4k_nb<CAI_Q4_K>>(p, gxs, n_slices, lds); else nb_launch<gemm_q4k_nb<CAI_Q5_K>>(p, gxs, n_slices, lds);
    } else {
      const size_t lds = (size_t)S * NB_SC * NB_LDX * 2 + (size_t)S * NB_TK * 4;
      const bool tail = p.cols % 256 != 0;
      if (qt == CAI_Q6_K && n_tok > NB_TK) nb_launch<gemm_q6k_nb<2>>(p, gxs, n_slices, 2 * lds);
      else if (qt == CAI_Q6_K) nb_launch<gemm_q6k_nb<1>>(p, gxs, n_slices, lds);
      else if (qt == CAI_Q8_0) { if (tail) nb_launch<gemm_blk_nb<CAI_Q8_0, true>>(p, gxs, n_slices, lds); else nb_launch<gemm_blk_nb<CAI_Q8_0, false>>(p, gxs, n_slices, lds); }
      else if (qt == CAI_I8ROW) { if (tail) nb_launch<gemm_blk_nb<CAI_I8ROW, true>>(p, gxs, n_slices, lds); else nb_launch<gemm_blk_nb<CAI_I8ROW, false>>(p, gxs, n_slices, lds); }
      else { if (tail) nb_launch<gemm_blk_nb<CAI_Q4_0, true>>(p, gxs, n_slices, lds); else nb_launch<gemm_blk_nb<CAI_Q4_0, false>>(p, gxs, n_slices, lds); }
    }
  }
  for (int i = 0; i < n_w; i++) g_prod.seg[i] = segs[i];
  g_prod.n_seg = n_w; g_prod.n_slices = n_slices; g_prod.n_tok = n_tok; g_prod.part_stride = stride; g_prod.width = width;
  g_prod.in_ssq = g_pending_ssq; g_prod.in_nsb = (g_pending_K + 255) >> 8; g_prod.in_K = g_pending_K; g_prod.in_eps = g_pending_eps;
  return CAI_OK;
}

// y <- last product (+bias, +residual), pending RMSNorm applied
int nb_reduce(float* y, int64_t y_stride, const float* residual)
{
  if (g_prod.n_seg < 1) return set_error(CAI_ERR_STATE, "small-batch reduce: no product in flight");
  NbReduceParams p{};
  for (int i = 0; i < 3; i++) p.seg[i] = g_prod.seg[i];
  p.n_seg = g_prod.n_seg; p.part = g_nb.part; p.part_stride = g_prod.part_stride; p.n_slices = g_prod.n_slices; p.n_tok = g_prod.n_tok;
  p.in_ssq = g_prod.in_ssq; p.in_nsb = g_prod.in_nsb; p.in_K = g_prod.in_K; p.in_eps = g_prod.in_eps;
  p.y = y; p.y_stride = y_stride; p.residual = residual; p.width = g_prod.width;
  hipLaunchKernelGGL(nb_reduce_kernel, dim3((p.width + 255) / 256, p.n_tok), dim3(256), 0, ctx().stream, p.part, (long long)p.part_stride, p.n_slices, p.n_tok, p.width, p);
  g_prod.n_seg = 0;
  return CAI_OK;
}

// Tokens one pass of nb_prep / nb_gemm / nb_reduce takes for this weight type
int nb_pass_tokens(const cai_qw_s* w) { return w->qtype == CAI_Q6_K ? NB_TMAX : NB_TK; }

// Whole linear layer, 8 tokens per pass (the weights are streamed once per pass): y = W (gain . x / rms) + bias (+ residual)
int nb_linear(const cai_qw_s* w, const float* x, int64_t x_stride, const float* gain, float eps, int n_tok, float* y, int64_t y_stride, const float* residual)
{
  int rc;
  // Q4_K matrices of whole row sets: the one-launch form (cai_gemm_ra.hip), 8 tokens per launch
  if (ra_supported(&w, 1, gain != nullptr, 0) && !(x_stride & 3) && !(y_stride & 3) && !(reinterpret_cast<uintptr_t>(x) & 15) && !(reinterpret_cast<uintptr_t>(y) & 15) &&
      !(residual && (reinterpret_cast<uintptr_t>(residual) & 15)) && !(gain && (reinterpret_cast<uintptr_t>(gain) & 15)) && !(w->bias && (reinterpret_cast<uintptr_t>(w->bias) & 15))) {
    if ((rc = ra_reserve(ra_part_floats(w->rows, w->cols)))) return rc;
    for (int t0 = 0; t0 < n_tok; t0 += 8) {
      const int zero = 0;
      if ((rc = ra_gemm(&w, &zero, 1, std::min(8, n_tok - t0), x + (int64_t)t0 * x_stride, x_stride, gain, eps, 0, y + (int64_t)t0 * y_stride, y_stride,
                        residual ? residual + (int64_t)t0 * y_stride : nullptr))) return rc;
    }
    return CAI_OK;
  }
  const int pass = nb_pass_tokens(w);
  if ((rc = nb_reserve((int)w->cols, (size_t)nb_max_slices((int)w->cols) * pass * ((w->rows + 3) / 4 * 4)))) return rc;
  for (int t0 = 0; t0 < n_tok; t0 += pass) {
    const int nt = std::min(pass, n_tok - t0); const int zero = 0;
    if ((rc = nb_prep_plain(x + (int64_t)t0 * x_stride, x_stride, gain, eps, (int)w->cols, nt))) return rc;
    if ((rc = nb_gemm(&w, &zero, 1, nt))) return rc;
    if ((rc = nb_reduce(y + (int64_t)t0 * y_stride, y_stride, residual ? residual + (int64_t)t0 * y_stride : nullptr))) return rc;
  }
  return CAI_OK;
}

}  // namespace cai
