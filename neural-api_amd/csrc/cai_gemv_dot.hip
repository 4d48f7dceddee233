// Persistent streaming matrix-vector kernel for batch-1 decode on gfx950, integer-dot form: Q4_K, and with other requests and
// block arithmetic in the same walk Q5_K (stored super-blocks), Q4_0 (quants and scales planes) and Q6_K (ql|qh records +
// planes of scales and d).
//
// The weights of a Q4_K sub-block are 4-bit integers with one float scale, so dot(W[a], X) splits into an exact
// integer part and a handful of float operations per 32 weights once X is held as integers too.  Each
// work-group turns the activation vector (token RMSNorm fused) into block-float form once: per 32 values one
// float scale s = max|x| / (2^22 - 1) and 23-bit integers q = rint(x / s), stored as three balanced base-256
// digits (each a signed byte).  The inner loop is then v_dot4_i32_i8 on nibbles widened to bytes: 3 mask/shift
// operations and 6 dot4 per 8 weights instead of 16 conversions + 16 FMAs.  The integer sums are exact; the
// only rounding beyond the float path is that of x itself, 2^-23 of its 32-block maximum.
//
// Work layout (as in the float kernel): a fixed number of work-groups stays resident and strides over the row
// groups; one lane owns one pair of sub-blocks (64 weights = two 128-bit loads + the 16-byte super-block
// header); rows longer than 4096 columns are split over `nsw` waves, each keeping its slice of the quantised
// activation in registers (52 VGPRs); widths of 17..24 super-blocks pack four rows into a wave instead (slices of four
// super-blocks), so that no lanes idle.  Weights of the next NS-1 row groups are in flight while one is reduced.
//
// Semantics: Out[a] = act(dot(W[a], X) + bias[a]) (+ residual), or for the fused feed-forward front half
// Out[i] = up_i * silu(gate_i) with up = row i and gate = row half + i
// (reference: neural/neuralvolume.pas:12127-12423; neural/neural.cl:111-146, 1047-1085, 1213-1263).
#include "cai_gemv_common.hpp"
#include <set>
#include <type_traits>

namespace cai {

namespace {

struct Q4kRegs { uint4 h, q0, q1; };
struct Q5kRegs { uint4 h, q0, q1, e0, e1; };   // Q5_K: + the 32 bytes of the fifth-bit plane (neural/neuralgguf.pas:516-587)
template <int QT> constexpr int dot_rec_bytes() { return QT == CAI_Q6_K ? 192 : QT == CAI_Q4_0 ? 128 : QT == CAI_Q5_K ? 176 : 144; }

// LDS slot (in uint4) of the t-th uint4 (t = 0..15) of unit u (64 activations): tiles of 16 units, transposed
__device__ __forceinline__ int xq_slot(int u, int t) { return (u >> 4) * 256 + t * 16 + (u & 15); }

constexpr float XQ_MAX = 4194303.0f;          // 2^22 - 1
constexpr int NL = 3;                         // balanced base-256 digits per activation

__device__ __forceinline__ float quad_max(float v)
{
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xb1, 0xf, 0xf, true)));  // quad_perm [1,0,3,2]
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4e, 0xf, 0xf, true)));  // quad_perm [2,3,0,1]
  return v;
}
__device__ __forceinline__ float quad_poison(float v)   // v is 0 or NaN per lane; NaN if any lane of the quad has it
{
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xb1, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4e, 0xf, 0xf, true));
  return v;
}
__device__ __forceinline__ int quad_sum(int v)
{
  v += __builtin_amdgcn_update_dpp(0, v, 0xb1, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x4e, 0xf, 0xf, true);
  return v;
}

// sum over each group of 64 / PK lanes, valid in the group's last lane
template <int PK>
__device__ __forceinline__ float group_sum(float v)
{
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, true)); // row_shr:1
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x112, 0xf, 0xf, true)); // row_shr:2
  if (PK <= 8) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, true)); // row_shr:4
  if (PK <= 4) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, true)); // row_shr:8
  if (PK <= 2) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, true)); // row_bcast:15
  return v;
}

// four rounded activations (as float bit patterns of x*inv + 1.5*2^23) -> one dword per digit
__device__ __forceinline__ void pack_digits(const float (&f)[4], int (&d)[NL])
{
  uint32_t e[4];
#pragma unroll
  for (int i = 0; i < 4; i++)   // integer value + 0x808080, then flip the digit sign bits: bytes are balanced digits
    e[i] = (__builtin_bit_cast(uint32_t, f[i]) + (0x00808080u - 0x4B400000u)) ^ 0x00808080u;
  const uint32_t p01 = __builtin_amdgcn_perm(e[1], e[0], 0x05010400u), p23 = __builtin_amdgcn_perm(e[3], e[2], 0x05010400u);
  const uint32_t h01 = __builtin_amdgcn_perm(e[1], e[0], 0x06020602u), h23 = __builtin_amdgcn_perm(e[3], e[2], 0x06020602u);
  d[0] = (int)__builtin_amdgcn_perm(p23, p01, 0x05040100u);
  d[1] = (int)__builtin_amdgcn_perm(p23, p01, 0x07060302u);
  d[2] = (int)__builtin_amdgcn_perm(h23, h01, 0x05040100u);
}

}  // namespace

// Q6_K in the same walk (neural/neuralgguf.pas:639-717; resident as 192-byte ql | qh records + planes of scales and d):
// the lane that owns activations 64 cc .. 64 cc + 63 of a super-block owns, in half nh = cc >> 1, the weights of j = 2 jp
// (its first 32 activations) and j = 2 jp + 1 (the second 32), jp = cc & 1: the low (jp = 0) or high nibbles of the two
// 32-byte ql runs and two of the four 2-bit fields of the 32 qh bytes.  Codes 0..63 go to v_dot4 as they are; the - 32
// offset uses the sums of the lane's integer activations per 16, taken once; each 16 weights have their own scale.
struct Q6kRegs { uint4 a0, a1, b0, b1, h0, h1; uint2 sc; uint32_t d; };

// PK > 1 packs PK rows into one wave: a wave then holds 16 / PK super-blocks of PK different row-group streams (lane
// quarter-groups of 64 / PK lanes), so a width that is not a multiple of 4096 columns leaves no lanes idle - 5120 columns
// are five waves of 4 super-blocks x 4 rows instead of two waves of 16 + 4 super-blocks x 1 row.  The row a lane works on
// then differs inside the wave (addresses and group indices are vector values), sums are taken per lane group and the
// outputs always finish through LDS.
// The arguments every work-group needs before it can issue its first requests travel as leading scalar kernel arguments:
// the compiler is told to have the first 14 dwords of the argument block preloaded into scalar registers at wave launch
// (-mllvm -amdgpu-kernarg-preload-count), so neither the activation requests nor the first weight requests wait for a round
// trip to the argument block (fields of the parameter struct are fetched where they are first used, one round trip each).
// rows0: rows of segment 0 (the fused feed-forward walk: the half); geo = waves along a row | waves (row streams) along the
// rows << 8 | slots of the sum-of-squares hand-off / 64 << 16.
struct DotHot { const float* x; const uint8_t* w0; const float* gain; const float* ssq_in; int cols, n_groups, geo, grid, rows0; };
#define DOT_HOT_ARGS const float* hx, const uint8_t* hw0, const float* hgain, const float* hssq, const int hcols, const int hgroups, const int hgeo, const int hgrid, const int hrows0
#define DOT_HOT_PACK DotHot{hx, hw0, hgain, hssq, hcols, hgroups, hgeo, hgrid, hrows0}

template <int R, int MODE, bool MULTISEG, int NS, int QT, int PK = 1>
__device__ __forceinline__ void gemv_dot_body(const GemvParams& p, const DotHot a)
{
  const int n_groups = a.n_groups, nsw = a.geo & 0xff, gwv = (a.geo >> 8) & 0xff, ssq_n = (a.geo >> 16) << 6;
  const int half = MODE == 1 ? a.rows0 : 0;
  const int nthr_wg = 64 * nsw * (gwv / PK);     // threads of the work-group (the launcher's geometry)
  extern __shared__ uint4 xq4[];
  const unsigned long long tl0 = timeline_now();
  constexpr int RR = MODE == 1 ? 2 * R : R;
  constexpr int TS = 16 / PK;                 // super-blocks of a row held by one wave
  static_assert(PK == 1 || PK == 2 || PK == 4 || PK == 8, "rows packed per wave");
  __shared__ float s_ss[16];
  constexpr int CH = 4;                       // row groups between two meetings of the slice waves
  __shared__ float s_part[2][16][CH][PK * RR];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: group indices, segment lookups and loop bounds stay scalar
  const int step = wave % nsw, gquad = wave / nsw;
  const int prow = PK > 1 ? (lane >> 2) / TS : 0;          // which of the wave's PK row streams this lane belongs to
  const int gslot = gquad * PK + prow;
  const int cols = a.cols, nsb = cols >> 8;
  const int64_t row_bytes = (int64_t)nsb * dot_rec_bytes<QT>();
  const int sb = step * TS + (PK > 1 ? (lane >> 2) % TS : (lane >> 2)), cc = lane & 3;
  const bool act = sb < nsb;
  const int g_first = blockIdx.x * gwv + gslot, g_stride = a.grid * gwv;
  const int n_iters = (n_groups + g_stride - 1) / g_stride;
  const int64_t lane_off = (int64_t)(act ? sb : 0) * dot_rec_bytes<QT>();
  using WRegs = typename std::conditional<QT == CAI_Q6_K, Q6kRegs, typename std::conditional<QT == CAI_Q5_K, Q5kRegs, Q4kRegs>::type>::type;

  // group -> segment, first row of the group inside the segment
  auto locate = [&](int g, const GemvSeg*& sg, int& row0) {
    int s = 0, g0 = 0;
    if (MULTISEG) {
      if (p.n_seg > 1 && g >= p.seg[0].grp_end) { s = 1; g0 = p.seg[0].grp_end; }
      if (p.n_seg > 2 && g >= p.seg[1].grp_end) { s = 2; g0 = p.seg[1].grp_end; }
    }
    sg = &p.seg[s]; row0 = (g - g0) * R;
  };
  // the same, with the weight pointer of segment 0 taken from the preloaded arguments
  auto locate_w = [&](int g, const uint8_t*& data, const uint8_t*& aux, int& rows, int& row0) {
    int s = 0, g0 = 0;
    if (MULTISEG) {
      if (p.n_seg > 1 && g >= p.seg[0].grp_end) { s = 1; g0 = p.seg[0].grp_end; }
      if (p.n_seg > 2 && g >= p.seg[1].grp_end) { s = 2; g0 = p.seg[1].grp_end; }
    }
    data = (!MULTISEG || s == 0) ? a.w0 : p.seg[s].data;
    if (QT == CAI_Q4_K || QT == CAI_Q5_K) aux = nullptr; else aux = p.seg[s].aux;
    rows = (!MULTISEG || s == 0) ? a.rows0 : p.seg[s].rows;
    row0 = (g - g0) * R;
  };
  // Loads are never conditional: past the last group the last one is fetched again, lanes beyond the row's width fetch
  // super-block 0 (both cache hits, the values are not used).  A load under a branch would make the compiler wait for
  // ALL outstanding loads wherever the paths join, i.e. before every new request.
  // the same with the group index a vector value (packed rows): the segment's fields are selected, not fetched through a
  // per-lane pointer (that would put a dependent load in front of every weight request)
  struct SegV { const uint8_t* data; const uint8_t* aux; int rows, row0; };
  auto locate_v = [&](int g) {
    SegV v{p.seg[0].data, p.seg[0].aux, p.seg[0].rows, 0};
    int g0 = 0;
    if (MULTISEG) {
      if (p.n_seg > 1 && g >= p.seg[0].grp_end) { v.data = p.seg[1].data; v.aux = p.seg[1].aux; v.rows = p.seg[1].rows; g0 = p.seg[0].grp_end; }
      if (p.n_seg > 2 && g >= p.seg[1].grp_end) { v.data = p.seg[2].data; v.aux = p.seg[2].aux; v.rows = p.seg[2].rows; g0 = p.seg[1].grp_end; }
    }
    v.row0 = (g - g0) * R;
    return v;
  };
  auto issue = [&](int g, WRegs (&rg)[RR]) {
    SegV sv;
    if constexpr (PK > 1) sv = locate_v(min(g, n_groups - 1));
    else locate_w(min(g, n_groups - 1), sv.data, sv.aux, sv.rows, sv.row0);
    const SegV* sg = &sv;
    const int row0 = sv.row0;
    const int lim = MODE == 1 ? half : sg->rows;
#pragma unroll
    for (int r = 0; r < RR; r++) {
      int row = row0 + (MODE == 1 ? (r >> 1) : r);
      if (row >= lim) row = lim - 1;               // tail group: re-read the last row, result is not written
      if (MODE == 1 && (r & 1)) row += half;
      const uint8_t* blk = sg->data + (int64_t)row * row_bytes + lane_off;
      if constexpr (QT == CAI_Q6_K) {
        const int nh = cc >> 1;
        const int64_t b = (int64_t)row * nsb + (act ? sb : 0);
        rg[r].a0 = *reinterpret_cast<const uint4*>(blk + 64 * nh);      rg[r].a1 = *reinterpret_cast<const uint4*>(blk + 64 * nh + 16);
        rg[r].b0 = *reinterpret_cast<const uint4*>(blk + 64 * nh + 32); rg[r].b1 = *reinterpret_cast<const uint4*>(blk + 64 * nh + 48);
        rg[r].h0 = *reinterpret_cast<const uint4*>(blk + 128 + 32 * nh); rg[r].h1 = *reinterpret_cast<const uint4*>(blk + 144 + 32 * nh);
        rg[r].sc = *reinterpret_cast<const uint2*>(sg->aux + b * 16 + 8 * nh);
        rg[r].d = *reinterpret_cast<const uint16_t*>(p.seg_aux2[0] + b * 2);   // (Q6_K launches hold one segment)
      } else if constexpr (QT == CAI_Q4_0) {
        // quants plane: the lane's two 32-weight blocks are 32 contiguous bytes; scales plane: their two halfs one dword
        rg[r].q0 = *reinterpret_cast<const uint4*>(blk + 32 * cc);
        rg[r].q1 = *reinterpret_cast<const uint4*>(blk + 32 * cc + 16);
        rg[r].h.x = *reinterpret_cast<const uint32_t*>(sg->aux + ((int64_t)row * nsb + (act ? sb : 0)) * 16 + 4 * cc);
      } else if constexpr (QT == CAI_Q5_K) {
        // header as Q4_K; the lane's 32 nibble bytes sit behind the 32-byte bit plane, which all four lanes of the super-block read
        rg[r].h = *reinterpret_cast<const uint4*>(blk);
        rg[r].e0 = *reinterpret_cast<const uint4*>(blk + 16); rg[r].e1 = *reinterpret_cast<const uint4*>(blk + 32);
        rg[r].q0 = *reinterpret_cast<const uint4*>(blk + 48 + 32 * cc);
        rg[r].q1 = *reinterpret_cast<const uint4*>(blk + 64 + 32 * cc);
      } else {
        rg[r].h = *reinterpret_cast<const uint4*>(blk);
        rg[r].q0 = *reinterpret_cast<const uint4*>(blk + 16 + 32 * cc);
        rg[r].q1 = *reinterpret_cast<const uint4*>(blk + 32 + 32 * cc);
      }
    }
  };

  WRegs buf[NS][RR];

  // ---- activation -> block-float integers, once per work-group, through LDS ----
  {
    float inv_rms = 1.0f;
    const float4* src = reinterpret_cast<const float4*>(a.x);
    const int n8 = cols >> 3, nthr = nthr_wg;
    // one thread = 8 consecutive activations (a quarter of a 32-block: the block's four threads are one DPP quad).
    // A thread's turns (n, n + nthr, ...) are requested SD at a time - a long row (the 18944-wide down projection: four
    // turns) costs one cache round trip instead of one per turn; the first batch goes out before the sum of squares.
    constexpr int SD = (MODE == 1 || MULTISEG) ? 1 : 4;   // (the fused-norm walks have rows of one turn; batching only costs them registers)
    typedef float f4 __attribute__((ext_vector_type(4)));   // (arrays of HIP's float4 struct end up in scratch memory)
    const f4* src4 = reinterpret_cast<const f4*>(a.x);
    const f4* gsrc4 = reinterpret_cast<const f4*>(a.gain);
    f4 c0[SD], c1[SD], cg0[SD], cg1[SD];
    auto request = [&](int n0) {
#pragma unroll
      for (int u = 0; u < SD; u++) {
        const int nn = min(n0 + u * nthr, n8 - 1);     // past the end: the last eight again (not used)
        c0[u] = src4[2 * nn]; c1[u] = src4[2 * nn + 1];
        if (a.gain) { cg0[u] = gsrc4[2 * nn]; cg1[u] = gsrc4[2 * nn + 1]; }
        else { cg0[u] = (f4)(0.0f); cg1[u] = (f4)(0.0f); }
      }
    };
    request(threadIdx.x);
    // Requests return in the order they were issued: the activation (and the producer's sum-of-squares partials) go out
    // BEFORE the first weight requests, so that their arrival does not queue behind the first burst of weights from HBM
    // and the block-float conversion runs while that burst is on its way (weights first: 605 tok/s on the 7B shape, this
    // order 618).
    float tq[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const bool ssq_short = a.gain && a.ssq_in && ssq_n <= 256;
    if (ssq_short) {
#pragma unroll
      for (int u = 0; u < 4; u++) tq[u] = a.ssq_in[min(u * 64 + lane, ssq_n - 1)];
    }
#pragma unroll
    for (int k = 0; k < NS - 1; k++) issue(g_first + k * g_stride, buf[k]);
    timeline_put(p.timeline, 0, tl0);
    timeline_stamp(p.timeline, 1);
    if (a.gain) {
      float t = 0.0f;
      if (a.ssq_in) {
        // sum of squares of x delivered by the producing kernel as SSQ_PARTS per-work-group partials (fixed order)
        if (ssq_short) {
#pragma unroll
          for (int u = 0; u < 4; u++) t += u * 64 < ssq_n ? tq[u] : 0.0f;
        } else
#pragma unroll 4
        for (int i = 0; i < ssq_n / 64; i++) t += a.ssq_in[i * 64 + lane];
        t = wave_sum(t);
        t = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, t), 63));
      } else {
        for (int k0 = threadIdx.x; k0 < n8 * 2; k0 += 4 * nthr) {      // four requests per turn, squares added in index order
          float4 v[4];
#pragma unroll
          for (int u = 0; u < 4; u++) v[u] = src[min(k0 + u * nthr, n8 * 2 - 1)];
#pragma unroll
          for (int u = 0; u < 4; u++)
            if (k0 + u * nthr < n8 * 2) { t = fmaf(v[u].x, v[u].x, t); t = fmaf(v[u].y, v[u].y, t); t = fmaf(v[u].z, v[u].z, t); t = fmaf(v[u].w, v[u].w, t); }
        }
        t = wave_sum(t);
        if (lane == 63) s_ss[wave] = t;
        __syncthreads();
        t = 0.0f;
        for (int w = 0; w < (nthr_wg >> 6); w++) t += s_ss[w];
        __syncthreads();                                 // s_ss is reused by the output sum of squares
      }
      inv_rms = 1.0f / sqrtf(t / (float)cols + p.norm_eps);
    }
    timeline_stamp_after(p.timeline, 2, c0[0].x + inv_rms);
    for (int n0 = threadIdx.x; n0 < n8; n0 += SD * nthr) {
     if (n0 != (int)threadIdx.x) request(n0);
#pragma unroll
     for (int t = 0; t < SD; t++) {
      const int n = n0 + t * nthr;
      if (n < n8) {
      f4 v0 = c0[t], v1 = c1[t];
      const f4 g0 = cg0[t], g1 = cg1[t];
      if (a.gain) {
        v0.x = g0.x * (v0.x * inv_rms); v0.y = g0.y * (v0.y * inv_rms); v0.z = g0.z * (v0.z * inv_rms); v0.w = g0.w * (v0.w * inv_rms);
        v1.x = g1.x * (v1.x * inv_rms); v1.y = g1.y * (v1.y * inv_rms); v1.z = g1.z * (v1.z * inv_rms); v1.w = g1.w * (v1.w * inv_rms);
      }
      float m = fmaxf(fmaxf(fmaxf(fabsf(v0.x), fabsf(v0.y)), fmaxf(fabsf(v0.z), fabsf(v0.w))),
                      fmaxf(fmaxf(fabsf(v1.x), fabsf(v1.y)), fmaxf(fabsf(v1.z), fabsf(v1.w))));
      m = quad_max(m);
      const bool ok = m > 0.0f && m < 3.0e38f;           // an all-zero block contributes 0
      // 0 for finite values, NaN when the eight hold an inf or a NaN: carried into the scale so the outputs show it
      const float poison = (((v0.x + v0.y) + (v0.z + v0.w)) + ((v1.x + v1.y) + (v1.z + v1.w))) * 0.0f;
      const float inv = ok ? XQ_MAX / m : 0.0f, s = ok ? m * (1.0f / XQ_MAX) : 0.0f;
      const float fa[4] = {fmaf(v0.x, inv, 12582912.0f), fmaf(v0.y, inv, 12582912.0f), fmaf(v0.z, inv, 12582912.0f), fmaf(v0.w, inv, 12582912.0f)};
      const float fb[4] = {fmaf(v1.x, inv, 12582912.0f), fmaf(v1.y, inv, 12582912.0f), fmaf(v1.z, inv, 12582912.0f), fmaf(v1.w, inv, 12582912.0f)};
      int da[NL], db[NL];
      pack_digits(fa, da); pack_digits(fb, db);
      int isum = 0;
#pragma unroll
      for (int i = 0; i < 4; i++)
        isum += (int)(__builtin_bit_cast(uint32_t, fa[i]) - 0x4B400000u) + (int)(__builtin_bit_cast(uint32_t, fb[i]) - 0x4B400000u);
      isum = quad_sum(isum);
      // n = [unit][half:1][j:2]: the unit's record holds per digit 4 uint4 (2 per 32-block), then one uint4 of
      // {scale A, scale B, s*sum A, s*sum B}
      const int u = n >> 3, hb = (n >> 2) & 1, j = n & 3;
      uint32_t* rec = reinterpret_cast<uint32_t*>(xq4);
#pragma unroll
      for (int L = 0; L < NL; L++) {
        uint32_t* dst = rec + (size_t)xq_slot(u, L * 4 + hb * 2 + (j >> 1)) * 4 + (j & 1) * 2;
        dst[0] = (uint32_t)da[L]; dst[1] = (uint32_t)db[L];
      }
      // the block's scale must be poisoned by any of its four threads
      const float s_blk = s + quad_poison(poison);
      if (j == 0) {
        float* fr = reinterpret_cast<float*>(rec + (size_t)xq_slot(u, NL * 4) * 4);
        fr[hb] = s_blk; fr[2 + hb] = s_blk * (float)isum;
      }
      }
     }
    }
    __syncthreads();
    timeline_stamp(p.timeline, 3);
  }
  int xq[NL][16];
  float sA = 0.0f, sB = 0.0f, mA = 0.0f, mB = 0.0f;
  if (act) {
    const int u = sb * 4 + cc;
#pragma unroll
    for (int L = 0; L < NL; L++) {
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const uint4 v = xq4[xq_slot(u, L * 4 + t)];
        xq[L][4 * t] = (int)v.x; xq[L][4 * t + 1] = (int)v.y; xq[L][4 * t + 2] = (int)v.z; xq[L][4 * t + 3] = (int)v.w;
      }
    }
    const uint4 v = xq4[xq_slot(u, NL * 4)];
    sA = __builtin_bit_cast(float, v.x); sB = __builtin_bit_cast(float, v.y);
    mA = __builtin_bit_cast(float, v.z); mB = __builtin_bit_cast(float, v.w);
  } else {
#pragma unroll
    for (int L = 0; L < NL; L++)
#pragma unroll
      for (int t = 0; t < 16; t++) xq[L][t] = 0;
  }

  float s16[4] = {0.0f, 0.0f, 0.0f, 0.0f};   // Q6_K: the lane's integer activations summed per 16 (first / second 32: groups 0, 1 / 2, 3)
  if constexpr (QT == CAI_Q6_K) {
#pragma unroll
    for (int gq = 0; gq < 4; gq++) {
      int tot = 0;
#pragma unroll
      for (int L = 0; L < NL; L++) {
        int t = 0;
#pragma unroll
        for (int w = 0; w < 4; w++) t = __builtin_amdgcn_sdot4(0x01010101, xq[L][4 * gq + w], t, false);
        tot += t << (8 * L);
      }
      s16[gq] = (float)tot;
    }
  }
  timeline_stamp(p.timeline, 4);
  float ssq_acc = 0.0f;   // squares of the outputs this thread wrote (for the consumer's RMSNorm)
  float keep[RR];         // finished totals of the last row groups, one group per lane
#pragma unroll
  for (int r = 0; r < RR; r++) keep[r] = 0.0f;
  auto process = [&](WRegs (&cur)[RR], WRegs (&nxt)[RR], int it) {
    const int g = g_first + it * g_stride;
    issue(g + (NS - 1) * g_stride, nxt);
    float acc[RR];
#pragma unroll
    for (int r = 0; r < RR; r++) acc[r] = 0.0f;
    if (PK > 1 || g < n_groups) {   // lanes beyond the row's width hold zero activations: they add exactly 0; packed rows: groups differ per lane, totals past the end are dropped below
#pragma unroll
      for (int r = 0; r < RR; r++) {
        if constexpr (QT == CAI_Q6_K) {
          const uint32_t qa[8] = {cur[r].a0.x, cur[r].a0.y, cur[r].a0.z, cur[r].a0.w, cur[r].a1.x, cur[r].a1.y, cur[r].a1.z, cur[r].a1.w};
          const uint32_t qb[8] = {cur[r].b0.x, cur[r].b0.y, cur[r].b0.z, cur[r].b0.w, cur[r].b1.x, cur[r].b1.y, cur[r].b1.z, cur[r].b1.w};
          const uint32_t qh[8] = {cur[r].h0.x, cur[r].h0.y, cur[r].h0.z, cur[r].h0.w, cur[r].h1.x, cur[r].h1.y, cur[r].h1.z, cur[r].h1.w};
          const int sh = 4 * (cc & 1);
          int ig[4][NL];
#pragma unroll
          for (int gq = 0; gq < 4; gq++)
#pragma unroll
            for (int L = 0; L < NL; L++) ig[gq][L] = 0;
#pragma unroll
          for (int w = 0; w < 8; w++) {
            const uint32_t hw = qh[w] >> sh;
            const int ca = (int)(((qa[w] >> sh) & 0x0f0f0f0fu) | ((hw << 4) & 0x30303030u));
            const int cb = (int)(((qb[w] >> sh) & 0x0f0f0f0fu) | ((hw << 2) & 0x30303030u));
#pragma unroll
            for (int L = 0; L < NL; L++) {
              ig[w >> 2][L] = __builtin_amdgcn_sdot4(ca, xq[L][w], ig[w >> 2][L], false);
              ig[2 + (w >> 2)][L] = __builtin_amdgcn_sdot4(cb, xq[L][8 + w], ig[2 + (w >> 2)][L], false);
            }
          }
          const uint32_t scw = (cc & 1) ? cur[r].sc.y : cur[r].sc.x;   // the four scales of this lane's groups, in order
          float fg[4];
#pragma unroll
          for (int gq = 0; gq < 4; gq++)
            fg[gq] = (float)(int)(int8_t)((scw >> (8 * gq)) & 0xffu) * fmaf(-32.0f, s16[gq], (float)ig[gq][0] + 256.0f * (float)ig[gq][1] + 65536.0f * (float)ig[gq][2]);   // (16 * 63 * 2^22 exceeds 32 bits: the digits are combined in float)
          const float d = __half2float(__ushort_as_half((unsigned short)cur[r].d));
          acc[r] = d * (sA * (fg[0] + fg[1]) + sB * (fg[2] + fg[3]));
          continue;
        } else if constexpr (QT == CAI_Q4_0) {
          // block A = q0 (low nibbles: weights 0..15, high: 16..31), block B = q1; x = d * (nibble - 8) (neural/neuralgguf.pas:811-845)
          const uint32_t qa[4] = {cur[r].q0.x, cur[r].q0.y, cur[r].q0.z, cur[r].q0.w}, qb[4] = {cur[r].q1.x, cur[r].q1.y, cur[r].q1.z, cur[r].q1.w};
          int ia[NL], ib[NL];
#pragma unroll
          for (int L = 0; L < NL; L++) { ia[L] = 0; ib[L] = 0; }
#pragma unroll
          for (int w = 0; w < 4; w++) {
            const int al = (int)(qa[w] & 0x0f0f0f0fu), ah = (int)((qa[w] >> 4) & 0x0f0f0f0fu);
            const int bl = (int)(qb[w] & 0x0f0f0f0fu), bh = (int)((qb[w] >> 4) & 0x0f0f0f0fu);
#pragma unroll
            for (int L = 0; L < NL; L++) {
              ia[L] = __builtin_amdgcn_sdot4(al, xq[L][w], ia[L], false);     ia[L] = __builtin_amdgcn_sdot4(ah, xq[L][4 + w], ia[L], false);
              ib[L] = __builtin_amdgcn_sdot4(bl, xq[L][8 + w], ib[L], false); ib[L] = __builtin_amdgcn_sdot4(bh, xq[L][12 + w], ib[L], false);
            }
          }
          const float fa = (float)(ia[0] + (ia[1] << 8) + (ia[2] << 16)), fb = (float)(ib[0] + (ib[1] << 8) + (ib[2] << 16));
          const float dA = __half2float(__ushort_as_half((unsigned short)(cur[r].h.x & 0xffffu)));
          const float dB = __half2float(__ushort_as_half((unsigned short)(cur[r].h.x >> 16)));
          acc[r] = dA * fmaf(sA, fa, -8.0f * mA) + dB * fmaf(sB, fb, -8.0f * mB);
          continue;
        } else if constexpr (QT == CAI_Q5_K) {
          // code = nibble | bit << 4 (0..31): bit 2 cc of plane byte i belongs to weight i of the first 32, bit 2 cc + 1 to the second
          const uint32_t qw[8] = {cur[r].q0.x, cur[r].q0.y, cur[r].q0.z, cur[r].q0.w, cur[r].q1.x, cur[r].q1.y, cur[r].q1.z, cur[r].q1.w};
          const uint32_t qe[8] = {cur[r].e0.x, cur[r].e0.y, cur[r].e0.z, cur[r].e0.w, cur[r].e1.x, cur[r].e1.y, cur[r].e1.z, cur[r].e1.w};
          int ia[NL], ib[NL];
#pragma unroll
          for (int L = 0; L < NL; L++) { ia[L] = 0; ib[L] = 0; }
#pragma unroll
          for (int w = 0; w < 8; w++) {
            const uint32_t ew = qe[w] >> (2 * cc);
            const int a = (int)((qw[w] & 0x0f0f0f0fu) | ((ew << 4) & 0x10101010u)), b = (int)(((qw[w] >> 4) & 0x0f0f0f0fu) | ((ew << 3) & 0x10101010u));
#pragma unroll
            for (int L = 0; L < NL; L++) {
              ia[L] = __builtin_amdgcn_sdot4(a, xq[L][w], ia[L], false);
              ib[L] = __builtin_amdgcn_sdot4(b, xq[L][8 + w], ib[L], false);
            }
          }
          // (32 * 31 * 2^22 exceeds 32 bits: the digits are combined in float)
          const float fa = (float)ia[0] + 256.0f * (float)ia[1] + 65536.0f * (float)ia[2], fb = (float)ib[0] + 256.0f * (float)ib[1] + 65536.0f * (float)ib[2];
          uint32_t sc, mn; q4k_scale_pair(cur[r].h.y, cur[r].h.z, cur[r].h.w, cc, sc, mn);
          const float d = __half2float(__ushort_as_half((unsigned short)(cur[r].h.x & 0xffffu)));
          const float dmin = __half2float(__ushort_as_half((unsigned short)(cur[r].h.x >> 16)));
          acc[r] = d * (cvt_ub0(sc) * (sA * fa) + cvt_ub1(sc) * (sB * fb)) - dmin * (cvt_ub0(mn) * mA + cvt_ub1(mn) * mB);
          continue;
        } else {
        const uint32_t qw[8] = {cur[r].q0.x, cur[r].q0.y, cur[r].q0.z, cur[r].q0.w, cur[r].q1.x, cur[r].q1.y, cur[r].q1.z, cur[r].q1.w};
        int ia[NL], ib[NL];
#pragma unroll
        for (int L = 0; L < NL; L++) { ia[L] = 0; ib[L] = 0; }
#pragma unroll
        for (int w = 0; w < 8; w++) {
          const int a = (int)(qw[w] & 0x0f0f0f0fu), b = (int)((qw[w] >> 4) & 0x0f0f0f0fu);
#pragma unroll
          for (int L = 0; L < NL; L++) {
            ia[L] = __builtin_amdgcn_sdot4(a, xq[L][w], ia[L], false);
            ib[L] = __builtin_amdgcn_sdot4(b, xq[L][8 + w], ib[L], false);
          }
        }
        const float fa = (float)(ia[0] + (ia[1] << 8) + (ia[2] << 16)), fb = (float)(ib[0] + (ib[1] << 8) + (ib[2] << 16));
        uint32_t sc, mn; q4k_scale_pair(cur[r].h.y, cur[r].h.z, cur[r].h.w, cc, sc, mn);
        const float d = __half2float(__ushort_as_half((unsigned short)(cur[r].h.x & 0xffffu)));
        const float dmin = __half2float(__ushort_as_half((unsigned short)(cur[r].h.x >> 16)));
        acc[r] = d * (cvt_ub0(sc) * (sA * fa) + cvt_ub1(sc) * (sB * fb)) - dmin * (cvt_ub0(mn) * mA + cvt_ub1(mn) * mB);
        }
      }
    }
    if constexpr (PK > 1) {
      // Packed rows: per-lane-group totals (last lane of each group), parked in LDS as the slice waves do, and one lane
      // per output row of the chunk finishes it.
      constexpr int SEGL = 64 / PK, RO = MODE == 1 ? R : RR;
      static_assert(CH * PK * RO <= 64, "one lane per output row of a chunk");
#pragma unroll
      for (int r = 0; r < RR; r++) acc[r] = group_sum<PK>(acc[r]);
      const int slot = it % CH, par = (it / CH) & 1;
      if ((lane & (SEGL - 1)) == SEGL - 1) {
#pragma unroll
        for (int r = 0; r < RR; r++) s_part[par][wave][slot][prow * RR + r] = acc[r];
      }
      if (slot != CH - 1 && it != n_iters - 1) return;
      __syncthreads();
      if (step != 0) return;
      const int n_out = (slot + 1) * PK * RO;
      if (lane >= n_out) return;
      const int sl = lane / (PK * RO), po = (lane / RO) % PK, r = lane % RO;
      const int gg = blockIdx.x * gwv + gquad * PK + po + (it - slot + sl) * g_stride;
      if (gg >= n_groups) return;
      const GemvSeg* sg; int row0; locate(gg, sg, row0);
      const int row = row0 + r;
      if (MODE == 0) {
        if (row >= sg->rows) return;
        float v = 0.0f;
        for (int s2 = 0; s2 < nsw; s2++) v += s_part[par][gquad * nsw + s2][sl][po * RR + r];
        if (sg->bias) v += sg->bias[row];
        v = act_apply(v, p.act);
        const int o = sg->y_off + row;
        if (p.residual) v += p.residual[o];
        p.y[o] = v; ssq_acc = fmaf(v, v, ssq_acc);
      } else {
        if (row >= p.half) return;
        float up = 0.0f, gate = 0.0f;
        for (int s2 = 0; s2 < nsw; s2++) { up += s_part[par][gquad * nsw + s2][sl][po * RR + 2 * r]; gate += s_part[par][gquad * nsw + s2][sl][po * RR + 2 * r + 1]; }
        if (sg->bias) { up += sg->bias[row]; gate += sg->bias[p.half + row]; }
        p.y[sg->y_off + row] = silu_mul(up, gate);
      }
      return;
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
        for (int s2 = 0; s2 < nsw; s2++) v += s_part[par][gquad * nsw + s2][sl][r];
        if (sg->bias) v += sg->bias[row];
        v = act_apply(v, p.act);
        const int o = sg->y_off + row;
        if (p.residual) v += p.residual[o];
        p.y[o] = v; ssq_acc = fmaf(v, v, ssq_acc);
      } else {
        if (row >= p.half) return;
        float up = 0.0f, gate = 0.0f;
        for (int s2 = 0; s2 < nsw; s2++) { up += s_part[par][gquad * nsw + s2][sl][2 * r]; gate += s_part[par][gquad * nsw + s2][sl][2 * r + 1]; }
        if (sg->bias) { up += sg->bias[row]; gate += sg->bias[p.half + row]; }
        p.y[sg->y_off + row] = silu_mul(up, gate);
      }
      return;
    }
    // One wave per row group: the totals of up to 16 groups are parked, one group per lane, and finished together
    // (bias, activation, residual, store: a single pass of vector code instead of one-lane code after every group).
    const int slot = it & 15;
#pragma unroll
    for (int r = 0; r < RR; r++) {
      const float tot = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc[r]), 63));
      keep[r] = lane == slot ? tot : keep[r];
    }
    if (slot != 15 && it != n_iters - 1) return;
    const int gg = g_first + (it - slot + lane) * g_stride;
    if (lane > slot || gg >= n_groups) return;
    const GemvSeg* sg; int row0; locate(gg, sg, row0);
    if (MODE == 0) {
#pragma unroll
      for (int r = 0; r < RR; r++) {
        const int row = row0 + r;
        if (row >= sg->rows) break;
        float v = keep[r];
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
        float up = keep[2 * r], gate = keep[2 * r + 1];
        if (sg->bias) { up += sg->bias[row]; gate += sg->bias[p.half + row]; }
        p.y[sg->y_off + row] = silu_mul(up, gate);
      }
    }
  };

  for (int it = 0; it < n_iters; it += NS) {
#pragma unroll
    for (int k = 0; k < NS; k++)
      if (it + k < n_iters) process(buf[k], buf[(k + NS - 1) % NS], it + k);
  }
  timeline_stamp(p.timeline, 5);

  if (p.ssq_out) {   // per-work-group partial of sum(y^2), summed in a fixed order; unused slots are zeroed by group 0
    __syncthreads();
    const float t = wave_sum(ssq_acc);
    if (lane == 63) s_ss[wave] = t;
    __syncthreads();
    if (threadIdx.x == 0) {
      float tot = 0.0f;
      for (int w = 0; w < (nthr_wg >> 6); w++) tot += s_ss[w];
      p.ssq_out[blockIdx.x] = tot;
    }
    if (blockIdx.x == 0) for (int i = a.grid + threadIdx.x; i < ssq_n; i += nthr_wg) p.ssq_out[i] = 0.0f;
  }
  timeline_stamp(p.timeline, 7);
}

template <int R, int MODE, bool MULTISEG, int NS, int PK = 1>
__global__ __launch_bounds__(768, 3) void gemv_q4k_dot(DOT_HOT_ARGS, const GemvParams p)
{
  gemv_dot_body<R, MODE, MULTISEG, NS, CAI_Q4_K, PK>(p, DOT_HOT_PACK);
}

template <int R, int MODE, bool MULTISEG, int NS, int PK = 1>
__global__ __launch_bounds__(768, 3) void gemv_q40_dot(DOT_HOT_ARGS, const GemvParams p)
{
  gemv_dot_body<R, MODE, MULTISEG, NS, CAI_Q4_0, PK>(p, DOT_HOT_PACK);
}

template <int R, int MODE, bool MULTISEG, int NS, int PK = 1>
__global__ __launch_bounds__(768, 3) void gemv_q5k_dot(DOT_HOT_ARGS, const GemvParams p)
{
  gemv_dot_body<R, MODE, MULTISEG, NS, CAI_Q5_K, PK>(p, DOT_HOT_PACK);
}

template <int R, int NS>
__global__ __launch_bounds__(768, 3) void gemv_q6k_dot(DOT_HOT_ARGS, const GemvParams p)
{
  gemv_dot_body<R, 0, false, NS, CAI_Q6_K>(p, DOT_HOT_PACK);
}

// Host launcher.  Returns CAI_ERR_UNSUPPORTED when the shape does not fit this kernel (caller falls back).
int launch_q4k_dot(GemvParams& p, const MultiGemv& m, int swiglu_half, hipStream_t st)
{
  Context& c = ctx();
  const int cols = p.cols, nsb = cols >> 8;
  int nsw = (nsb + 15) >> 4;                // waves along the columns
  if (nsw > 8 || cols % 256) return CAI_ERR_UNSUPPORTED;  // rows longer than 32768 columns; Q4_0 widths that are not whole 256-blocks
  const bool q6k = m.w[0]->qtype == CAI_Q6_K;
  if (q6k && (swiglu_half || m.n != 1)) return CAI_ERR_UNSUPPORTED;
  constexpr int W = 12;   // resident waves per CU
  // Rows packed per wave: a width of 17..24 super-blocks, whose second 4096-column slice would be mostly empty (5120 columns:
  // 20 of 32 lane quads at work), is cut into five or six slices of 4 super-blocks instead, four rows to a wave.  Measured
  // on 55296 x 5120: 40.7 -> 32.5 us, 6144 columns 42.9 -> 38.2; widths that fill one wave lose to the exchange through LDS
  // (2048 columns: 4.2 -> 4.9 us, 3584: 18.1 -> 19.6) and keep one row per wave.
  constexpr int PKW = 4;
  const bool packed = !q6k && nsb > 16 && nsb <= 24;
  if (packed) nsw = (nsb + 16 / PKW - 1) / (16 / PKW);
  // waves per work-group: short rows (one or two waves span the columns) use ONE work-group of 8 waves per CU - the
  // activation is quantised once per CU instead of once per 4 waves, which outweighs the lower wave count (measured:
  // 3 work-groups of 4 waves 537 tok/s, 1 of 12 waves 544, 1 of 8 waves 561 on the 7B shape); long rows fill the CU
  // with a single work-group of up to 12 waves
  int gwv = nsw >= 3 ? std::max(1, W / nsw) : 8 / nsw;   // the kernel is built for at most 12 waves per work-group
  int gquads = gwv;                                        // waves along the rows
  if (packed) { gquads = W / nsw; gwv = gquads * PKW; }   // two waves along the rows (one measured 6 % slower)
  int64_t total = 0;
  for (int i = 0; i < m.n; i++) total += swiglu_half ? swiglu_half : m.rows[i];
  const int waves_per_wg = nsw * gquads;
  const size_t lds = (size_t)((cols + 1023) / 1024 * 1024) * 4;   // 16 uint4 per 64 activations
  int wg_per_cu = W / waves_per_wg; if (wg_per_cu < 1) wg_per_cu = 1;
  { const int lds_fit = (int)((160 * 1024 - 4096) / (lds + 1024)); if (wg_per_cu > lds_fit) wg_per_cu = lds_fit < 1 ? 1 : lds_fit; }
  const int max_wgs = c.n_cu * wg_per_cu;
  // Two rows per group halve the turns of a wave and double what it has in flight.  With long rows (three or more waves
  // per row, every wave's lanes full) that only pays when the turns come out even - 7B down projection: 7 turns of one row
  // beat 4 of two, 570 -> 580 tok/s; with one or two waves per row two rows measured better even at uneven turns (32B
  // q|k|v and o: 136.9 against 134.1 tok/s).
  int R = 1;
  if (!swiglu_half && total >= (int64_t)max_wgs * gwv * 4) {
    const int64_t slots = (int64_t)max_wgs * gwv;
    const int64_t turns1 = (total + slots - 1) / slots, turns2 = ((total + 1) / 2 + slots - 1) / slots;
    if (nsw < 3 || 2 * turns2 <= turns1) R = 2;
    if (packed) R = 2;
  }
  if (q6k) R = 1;   // (two rows of Q6_K requests in flight twice over do not fit the registers)
  int cum = 0;
  for (int i = 0; i < m.n; i++) {
    const int64_t rows = swiglu_half ? swiglu_half : m.rows[i];
    cum += (int)((rows + R - 1) / R);
    p.seg[i].grp_end = cum;
  }
  // sum-of-squares hand-off: producer and consumer agree on the slots in use (one work-group per CU is what every geometry
  // above launches; a larger grid is cut to the slot count)
  p.ssq_n = std::min(SSQ_PARTS, (c.n_cu + 63) / 64 * 64);
  const int grid = std::min(std::min((cum + gwv - 1) / gwv, max_wgs), p.ssq_n);
  const dim3 block(64 * waves_per_wg);
  p.timeline = timeline_next(grid);
  auto go = [&](auto kern) {
    static std::set<const void*> raised;   // kernels whose dynamic-LDS limit has been raised
    // (a failing attribute call would leave a sticky error that a later hipGetLastError reports against an innocent launch)
    if (raised.insert((const void*)kern).second && hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 2048) != hipSuccess)
      (void)hipGetLastError();
    hipLaunchKernelGGL(kern, dim3(grid), block, lds, st, p.x, p.seg[0].data, p.norm_gain, p.ssq_in, p.cols, cum, nsw | gwv << 8 | (p.ssq_n >> 6) << 16,
                       grid, swiglu_half ? swiglu_half : p.seg[0].rows, p);
  };
  auto pick_pk = [&](auto ns, auto pk) {
    constexpr int NSV = decltype(ns)::value, PKV = decltype(pk)::value;
    if (m.w[0]->qtype == CAI_Q4_0) {
      if (swiglu_half) go(gemv_q40_dot<1, 1, false, NSV, PKV>);
      else if (m.n > 1) { if (R == 2) go(gemv_q40_dot<2, 0, true, NSV, PKV>); else go(gemv_q40_dot<1, 0, true, NSV, PKV>); }
      else { if (R == 2) go(gemv_q40_dot<2, 0, false, NSV, PKV>); else go(gemv_q40_dot<1, 0, false, NSV, PKV>); }
    }
    else if (m.w[0]->qtype == CAI_Q5_K) {
      if (swiglu_half) go(gemv_q5k_dot<1, 1, false, NSV, PKV>);
      else if (m.n > 1) { if (R == 2) go(gemv_q5k_dot<2, 0, true, NSV, PKV>); else go(gemv_q5k_dot<1, 0, true, NSV, PKV>); }
      else { if (R == 2) go(gemv_q5k_dot<2, 0, false, NSV, PKV>); else go(gemv_q5k_dot<1, 0, false, NSV, PKV>); }
    }
    else if (swiglu_half) go(gemv_q4k_dot<1, 1, false, NSV, PKV>);
    else if (m.n > 1) { if (R == 2) go(gemv_q4k_dot<2, 0, true, NSV, PKV>); else go(gemv_q4k_dot<1, 0, true, NSV, PKV>); }
    else { if (R == 2) go(gemv_q4k_dot<2, 0, false, NSV, PKV>); else go(gemv_q4k_dot<1, 0, false, NSV, PKV>); }
  };
  auto pick = [&](auto ns) {
    constexpr int NSV = decltype(ns)::value;
    if (q6k) go(gemv_q6k_dot<1, NSV>);
    else if (packed) pick_pk(ns, std::integral_constant<int, PKW>());
    else pick_pk(ns, std::integral_constant<int, 1>());
  };
  pick(std::integral_constant<int, 2>());   // two row groups per wave: one in flight while one is reduced (three or four, also for the one-row walks alone, measured slower on every shape)
  return CAI_OK;
}

}  // namespace cai
