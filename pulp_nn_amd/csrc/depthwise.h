// Depthwise convolution kernels: CHW input, [ch][ky][kx] weights, HWC output,
// exactly the layouts of the reference API
// (32bit/src/pulp_nn_depthwise_generic.c:74-81,179 and
//  pulp_nn_depthwise_3x3_s1.c:79-85,110,145-146).
//
// These are bandwidth-bound VALU kernels (9 MACs per output byte), not MFMA
// work.  One workgroup handles one image, one group of CG channels and one
// band of RB output rows:
//   1. stage: the (RB-1)*sy+ky input rows of every channel of the group are
//      copied from HBM into LDS with loads that run along x and on through the
//      following rows (the rows of a band are contiguous in a CHW plane).  Bytes
//      are stored as a ^ 0x80 (a - 128 as int8) and everything outside the image
//      (left / right / top / bottom padding) is stored as 0x80, so the compute
//      phase has no border cases.  128 * sum(w) is added back per channel.
//   2. compute: lane <-> channel.  The LDS channel stride is an odd number of
//      dwords, so the 64 lanes of a wave read 64 different banks.  For 3x3 a
//      lane produces 4 horizontally adjacent outputs per step from 3 (stride 1)
//      or 4 (stride 2) dwords per input row with v_dot4_i32_i8 on byte windows,
//      the reference's own trick (pulp_nn_depthwise_3x3_s1.c:89-91,154-159)
//      of using the filter (K0,K1,K2,0) and its shifted copy (0,K0,K1,K2).
//   3. store: a 4x4 byte transpose inside each lane quad (DPP + v_perm) turns
//      "4 pixels of my channel" into "4 channels of one pixel", so that 16
//      quads write 64 contiguous bytes of an HWC pixel.
#pragma once
#include <type_traits>

#include "memops.h"
#include "requant.h"


struct DwGeom {
  const uint8_t *in;
  const int8_t *wt;
  const int8_t *bias;  // may be null
  uint8_t *out;
  int B, CH, H, W, Ho, Wo;
  int kx, ky, pt, pl, sx, sy;
  int RB;       // output rows per band
  int NR;       // staged input rows per band: (RB-1)*sy + ky
  int LP;       // left pad columns in LDS (multiple of 4, >= pl)
  int LWD;      // LDS row stride in dwords
  int CSD;      // LDS channel stride in dwords (odd)
  int bands;    // ceil(Ho / RB)
  int cgroups;  // ceil(CH / CG)
  int total;    // B * bands * cgroups workgroups
  // increments of (dword, row, channel) when the staging slot index grows by 256
  int inc_dw, inc_row, inc_c;
  int in_align4;  // input pointer and W are multiples of 4: aligned dword loads are safe
  int out_vec4;   // output pointer and CH are multiples of 4: dword stores are safe
  // Packing of layers with fewer than 64 channels (dw3x3_lin_kernel only): CH and B describe the
  // input re-read as images of 64 planes (CHW images lie back to back, so that is the same memory);
  // CHR is the real channel count, planes the real number of planes B_real * CHR.
  int CHR;
  long long planes;
};

#define DW_CG 64  // channels per workgroup (one per lane)

__device__ __forceinline__ int dw_xcd_remap(int id, int total)
{
  const int q = total >> 3, rem = total & 7;
  const int x = id & 7, s = id >> 3;
  return x * q + min(x, rem) + s;
}

// Stage the input band of this workgroup into LDS (see step 1 above).
__device__ __forceinline__ void dw_stage(const DwGeom &g, unsigned *lds, const uint8_t *img, int c0, int iy_start)
{
  const int tid = threadIdx.x;
  const int slots = DW_CG * g.NR * g.LWD;
  int dw = tid % g.LWD;
  int t2 = tid / g.LWD;
  int row = t2 % g.NR;
  int c = t2 / g.NR;
  for (int s = tid; s < slots; s += 256) {
    unsigned v = 0;
    const int ch = c0 + c;
    const int iy = iy_start + row;
    const int ix = 4 * dw - g.LP;
    if (ch < g.CH && (unsigned)iy < (unsigned)g.H && ix + 3 >= 0 && ix < g.W) {
      const uint8_t *src = img + ((long long)ch * g.H + iy) * g.W + ix;
      if (g.in_align4 && ix >= 0 && ix + 3 < g.W) {
        v = *(const unsigned *)src;
      } else {
#pragma unroll
        for (int j = 0; j < 4; j++)
          if ((unsigned)(ix + j) < (unsigned)g.W) v |= (unsigned)src[j] << (8 * j);
      }
    }
    lds[c * g.CSD + row * g.LWD + dw] = v ^ 0x80808080u;
    dw += g.inc_dw;
    if (dw >= g.LWD) { dw -= g.LWD; row++; }
    row += g.inc_row;
    if (row >= g.NR) { row -= g.NR; c++; }
    c += g.inc_c;
  }
}

// 4x4 byte transpose across the four lanes of a quad: in: byte j of lane q =
// element (q, j); out: byte q' of lane j' = element (q', j').
__device__ __forceinline__ unsigned quad_transpose4x4(unsigned v, int lane)
{
  // exchange 16-bit halves with lane ^ 2
  unsigned t = (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0x4E /* quad_perm [2,3,0,1] */, 0xF, 0xF, true);
  v = (lane & 2) ? ((t >> 16) | (v & 0xFFFF0000u)) : ((v & 0x0000FFFFu) | (t << 16));
  // exchange bytes with lane ^ 1
  t = (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, true);
  v = (lane & 1) ? (((t >> 8) & 0x00FF00FFu) | (v & 0xFF00FF00u)) : ((v & 0x00FF00FFu) | ((t << 8) & 0xFF00FF00u));
  return v;
}

// The same transpose with v_perm_b32: sel1 / sel2 are per-lane byte selectors
// (quad_sel1 / quad_sel2 of the lane), so there is no per-lane branch or select.
// v_perm_b32 D, S0, S1, sel: selector values 0-3 pick bytes of S1, 4-7 bytes of S0.
__device__ __forceinline__ unsigned quad_sel1(int lane) { return (lane & 2) ? 0x03020706u : 0x05040100u; }
__device__ __forceinline__ unsigned quad_sel2(int lane) { return (lane & 1) ? 0x03070105u : 0x06020400u; }
__device__ __forceinline__ unsigned quad_transpose4x4_perm(unsigned v, unsigned sel1, unsigned sel2)
{
  unsigned t = (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0x4E /* quad_perm [2,3,0,1] */, 0xF, 0xF, true);
  v = __builtin_amdgcn_perm(t, v, sel1);
  t = (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, true);
  return __builtin_amdgcn_perm(t, v, sel2);
}

// bytes [o, o+4) of the little-endian byte string formed by the dwords of `span`
template <int O, int NS>
__device__ __forceinline__ unsigned dw_window(const unsigned (&span)[NS])
{
  constexpr int d = O / 4, sh = O % 4;
  if constexpr (sh == 0) return span[d];
  else if constexpr (d + 1 < NS) return __builtin_amdgcn_alignbyte(span[d + 1], span[d], sh);
  else return span[d] >> (8 * sh);
}

// acc += K0*byte[O] + K1*byte[O+1] + K2*byte[O+2] of the span; wA = (K0,K1,K2,0),
// wB = (0,K0,K1,K2) saves the byte alignment when the window starts at byte 1.
template <int O, int NS>
__device__ __forceinline__ void dw_tap(const unsigned (&span)[NS], unsigned wA, unsigned wB, int &acc)
{
  if constexpr (O % 4 == 1) acc = __builtin_amdgcn_sdot4((int)span[O / 4], (int)wB, acc, false);
  else acc = __builtin_amdgcn_sdot4((int)dw_window<O, NS>(span), (int)wA, acc, false);
}

// The first tap of an accumulator: start + K . window.  Asking for the saturating form selects the three-address
// dot instruction, which takes the start value as an operand of its own; the accumulate-in-place form the compiler
// otherwise prefers needs a register copy of the start value first.  Nothing here can reach the int32 range
// (|sum| < 2^21 plus the start value), so saturation never acts.
template <int O, int NS>
__device__ __forceinline__ int dw_tap_first(const unsigned (&span)[NS], unsigned wA, unsigned wB, int start)
{
  if constexpr (O % 4 == 1) return __builtin_amdgcn_sdot4((int)span[O / 4], (int)wB, start, true);
  else return __builtin_amdgcn_sdot4((int)dw_window<O, NS>(span), (int)wA, start, true);
}

// 3x3 depthwise, stride S (1 or 2) in both directions, left padding PL (0 or 1).
template <int S, int PL, int MODE>
__global__ __launch_bounds__(256) void dw3x3_kernel(DwGeom g, EpiArgs e)
{
  extern __shared__ unsigned dw_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  int id = dw_xcd_remap(blockIdx.x, g.total);
  const int cg = id % g.cgroups;
  id /= g.cgroups;
  const int band = id % g.bands;
  const int b = id / g.bands;
  const int c0 = cg * DW_CG;
  const int oy0 = band * g.RB;
  const int rows = min(g.RB, g.Ho - oy0);

  const uint8_t *img = g.in + (long long)b * g.CH * g.H * g.W;
  dw_stage(g, dw_lds, img, c0, oy0 * S - g.pt);

  // per-lane channel constants
  const int ch = c0 + lane;
  const bool ch_ok = ch < g.CH;
  unsigned wA[3], wB[3];  // (K0,K1,K2,0) and (0,K0,K1,K2) per filter row
  int corr = 0;
  bn_t kk = 0, ll = 0;
  if (ch_ok) {
    int wsum = 0;
#pragma unroll
    for (int i = 0; i < 3; i++) {
      const int8_t *p = g.wt + (long long)ch * 9 + 3 * i;
      const unsigned k0 = (uint8_t)p[0], k1 = (uint8_t)p[1], k2 = (uint8_t)p[2];
      wA[i] = k0 | (k1 << 8) | (k2 << 16);
      wB[i] = wA[i] << 8;
      wsum += (int)p[0] + (int)p[1] + (int)p[2];
    }
    corr = 128 * wsum + (g.bias ? (int)g.bias[ch] : 0);
    if (MODE == EPI_BN) {
      kk = e.k[ch];
      ll = e.lambda[ch];
    }
  } else {
#pragma unroll
    for (int i = 0; i < 3; i++) wA[i] = wB[i] = 0;
  }
  __syncthreads();

  // dwords per input row needed for 4 outputs: window j starts at byte
  // (4 - PL) + S*j of the span that begins one dword left of output column 4*xg*S
  constexpr int O0 = 4 - PL;
  constexpr int NS = (O0 + 3 * S + 2) / 4 + 1;
  const int xgroups = (g.Wo + 3) >> 2;
  const int items = rows * xgroups;
  const unsigned *lbase = dw_lds + lane * g.CSD + (g.LP >> 2) - 1;
  uint8_t *obase = g.out + (((long long)b * g.Ho + oy0) * g.Wo) * g.CH + c0;

  for (int it = wave; it < items; it += 4) {
    const int r = it / xgroups, xg = it - r * xgroups;
    int acc[4] = {corr, corr, corr, corr};
#pragma unroll
    for (int i = 0; i < 3; i++) {
      const unsigned *p = lbase + (r * S + i) * g.LWD + xg * S;
      unsigned span[NS];
#pragma unroll
      for (int d = 0; d < NS; d++) span[d] = p[d];
      dw_tap<O0, NS>(span, wA[i], wB[i], acc[0]);
      dw_tap<O0 + S, NS>(span, wA[i], wB[i], acc[1]);
      dw_tap<O0 + 2 * S, NS>(span, wA[i], wB[i], acc[2]);
      dw_tap<O0 + 3 * S, NS>(span, wA[i], wB[i], acc[3]);
    }
    unsigned packed = 0;
#pragma unroll
    for (int j = 0; j < 4; j++)
      packed |= (unsigned)requant<MODE>(acc[j], kk, ll, e.mult, e.shift) << (8 * j);
    // lane now holds 4 pixels of its channel; after the transpose it holds 4
    // channels (those of its quad) of pixel 4*xg + (lane & 3)
    packed = quad_transpose4x4(packed, lane);
    const int ox = 4 * xg + (lane & 3);
    const int cq = lane & ~3;
    if (ox < g.Wo) {
      uint8_t *o = obase + ((long long)r * g.Wo + ox) * g.CH + cq;
      if (g.out_vec4 && c0 + cq + 3 < g.CH) {
        *(unsigned *)o = packed;
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++)
          if (c0 + cq + c < g.CH) o[c] = (uint8_t)(packed >> (8 * c));
      }
    }
  }
}

// One group of 4 output columns of one channel per lane, walked down the rows of a band.
struct DwColumn {
  const unsigned *p;  // LDS: first dword of the window in the first staged row
  uint8_t *o;         // output byte of the first row for this lane (after the quad transpose)
  long long row_bytes;
  int LWD, dc0, rows;
  int corr, mult, shift;
  bn_t k, lambda;
  unsigned wA[3], wB[3], sel1, sel2;
  int store, nbytes;
};

// XR: LDS holds the raw input bytes and the ^ 0x80 is applied as a dword is read (the LDS-direct staging of
// dw3x3_lin_kernel cannot apply it).
template <int S, int PL, int MODE, bool FULL, bool EDGE, bool FASTQ, bool XR = false>
__device__ __forceinline__ void dw3x3_column(DwColumn c)
{
  constexpr int O0 = 4 - PL;
  constexpr int NS = (O0 + 3 * S + 2) / 4 + 1;
  bool in_row[NS];
#pragma unroll
  for (int d = 0; d < NS; d++) in_row[d] = !EDGE || (c.dc0 + d >= 0 && c.dc0 + d < c.LWD);
  // fetch() requests a row's dwords from LDS, finish() turns them into the window bytes; a row is fetched one
  // step before it is used, so that the LDS latency is covered by the arithmetic of the row before
  auto fetch = [&](unsigned (&raw)[NS]) {
#pragma unroll
    for (int d = 0; d < NS; d++) raw[d] = in_row[d] ? c.p[d] : (XR ? 0u : 0x80808080u);
    c.p += c.LWD;
  };
  auto finish = [&](const unsigned (&raw)[NS], unsigned (&span)[NS]) {
#pragma unroll
    for (int d = 0; d < NS; d++) span[d] = XR ? raw[d] ^ 0x80808080u : raw[d];
  };
  auto read_row = [&](unsigned (&span)[NS]) {
    unsigned raw[NS];
    fetch(raw);
    finish(raw, span);
  };
  // K_i . window_j of one input row, for the four output columns j
  auto taps = [&](const unsigned (&span)[NS], int i, int (&acc)[4]) {
    dw_tap<O0, NS>(span, c.wA[i], c.wB[i], acc[0]);
    dw_tap<O0 + S, NS>(span, c.wA[i], c.wB[i], acc[1]);
    dw_tap<O0 + 2 * S, NS>(span, c.wA[i], c.wB[i], acc[2]);
    dw_tap<O0 + 3 * S, NS>(span, c.wA[i], c.wB[i], acc[3]);
  };
  auto taps_first = [&](const unsigned (&span)[NS], int (&acc)[4]) {
    acc[0] = dw_tap_first<O0, NS>(span, c.wA[0], c.wB[0], c.corr);
    acc[1] = dw_tap_first<O0 + S, NS>(span, c.wA[0], c.wB[0], c.corr);
    acc[2] = dw_tap_first<O0 + 2 * S, NS>(span, c.wA[0], c.wB[0], c.corr);
    acc[3] = dw_tap_first<O0 + 3 * S, NS>(span, c.wA[0], c.wB[0], c.corr);
  };
  auto emit = [&](int (&acc)[4]) {
    unsigned packed = requant4_same<MODE, FASTQ>(acc[0], acc[1], acc[2], acc[3], c.k, c.lambda, c.mult, c.shift);
    packed = quad_transpose4x4_perm(packed, c.sel1, c.sel2);
    if constexpr (FULL) {
      *(unsigned *)c.o = packed;
    } else {
      if (c.store == 0) {
        *(unsigned *)c.o = packed;
      } else if (c.store == 1) {
        for (int j = 0; j < c.nbytes; j++) c.o[j] = (uint8_t)(packed >> (8 * j));
      }
    }
    c.o += c.row_bytes;
  };

  unsigned span[NS];
  if constexpr (S == 1) {
    // P: output row y-2 so far (K0, K1 rows done); Q: output row y-1 so far (K0 done)
    int P[4], Q[4];
    read_row(span);
    taps_first(span, P);
    read_row(span);
    taps(span, 1, P);
    taps_first(span, Q);
    // Three accumulator sets take the roles (finishing, middle, starting) in turn; the
    // loop is unrolled by three so that the hand-over costs no register moves.
    int R[4];
    unsigned nxt[NS];
    if (c.rows > 0) fetch(nxt);
    auto step = [&](int (&fin)[4], int (&mid)[4], int (&beg)[4], bool more) {
      finish(nxt, span);
      if (more) fetch(nxt);
      taps(span, 2, fin);
      emit(fin);
      taps(span, 1, mid);
      taps_first(span, beg);
    };
    for (int r = 0; c.rows > 0;) {
      step(P, Q, R, r + 1 < c.rows);
      if (++r >= c.rows) break;
      step(Q, R, P, r + 1 < c.rows);
      if (++r >= c.rows) break;
      step(R, P, Q, r + 1 < c.rows);
      if (++r >= c.rows) break;
    }
  } else {
    // Q: next output row so far (K0 row done)
    int Q[4];
    read_row(span);
    taps_first(span, Q);
    for (int r = 0; r < c.rows; r++) {
      read_row(span);
      taps(span, 1, Q);
      read_row(span);
      taps(span, 2, Q);
      emit(Q);
      taps_first(span, Q);
    }
  }
}

// 3x3 depthwise, fast variant for W % 4 == 0 and a 16-byte aligned input.
//
// LDS holds the band exactly as it lies in memory (rows of W bytes back to back,
// no column padding), so staging is a linear copy: each wave copies the
// contiguous run of each of its 16 channels with one 16-byte load per lane, all
// loads in flight before the first LDS write.  The columns left of 0 and right
// of W-1 are supplied in the compute phase instead: a wave works on one group of
// 4 output columns at a time and walks down the rows of the band, so whether a
// dword of the 3-dword window lies outside the row is decided once per column
// group; outside dwords are replaced by 0x80808080 (a = 0).  Walking down the rows
// also means every input dword is read from LDS once, not three times: the three
// partial sums an input row contributes to are kept in registers.
//
// FULL: Wo % 4 == 0, CH % 64 == 0 and the output is 4-byte aligned, so every lane
// stores one dword per output row without any bounds check.
#ifndef DW_WAVES
#define DW_WAVES 8  // waves per workgroup of dw3x3_lin_kernel
#endif
// DMA (FULL only; the host checks that byte offsets fit 31 bits and that the channel stride leaves room
// for a band's last 16-byte piece): the band is staged with buffer loads that write LDS directly, one
// instruction per channel, instead of through registers (no staging registers, no LDS stores with their
// bank conflicts, no VALU work); LDS then holds raw bytes and the ^ 0x80 is applied as a dword is read.
template <int S, int PL, int MODE, bool FULL, bool DMA = false>
__global__ __launch_bounds__(64 * DW_WAVES) void dw3x3_lin_kernel(DwGeom g, EpiArgs e)
{
  static_assert(!DMA || FULL, "LDS-direct staging only for whole 64-channel groups");
  constexpr int NWV = DW_WAVES, CPW = DW_CG / NWV;  // waves, channels staged per wave
  extern __shared__ unsigned dw_lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int id = dw_xcd_remap(blockIdx.x, g.total);
  const int cg = id % g.cgroups;
  id /= g.cgroups;
  const int band = id % g.bands;
  const int b = id / g.bands;
  const int c0 = cg * DW_CG;
  const int oy0 = band * g.RB;
  const int rows = min(g.RB, g.Ho - oy0);
  const int iy_start = oy0 * S - g.pt;
  const int LWD = g.LWD;  // = W / 4
  const int dummy = DW_CG * g.CSD;  // one spare dword behind the tile: target of masked-off writes

  // ---- stage -----------------------------------------------------------------
  const int r_lo = max(0, -iy_start), r_hi = min(g.NR, g.H - iy_start);  // rows of the band inside the image
  const int run_len = max(r_hi - r_lo, 0) * g.W;                        // bytes per channel
  const bool two = run_len + 12 > 64 * 16;  // a run may need more than 64 chunks
  if constexpr (DMA) {
    // Lane l fetches the 16-byte chunk l of a channel's band (dwords 4l .. 4l+3).  Dwords [lo_d, hi_d) lie inside
    // the image; a chunk wholly outside is requested out of range (zeros); a chunk that straddles the first or last
    // image row is left out and fetched dword by dword (runs of 64 dwords q1 / q2).
    typedef __attribute__((address_space(3))) void *lds_ptr_t;
    const unsigned OOB = 0x80000000u;
    const __amdgpu_buffer_rsrc_t rsrc_in =
        __builtin_amdgcn_make_buffer_rsrc((void *)g.in, 0, (unsigned)(g.planes * g.H * g.W), 0x00020000);
    const int nchunks = (g.NR * LWD + 3) >> 2;
    const int lo_d = r_lo * LWD, hi_d = r_hi * LWD;
    const int hi_e = r_hi == g.NR ? 0x7fffffff : hi_d;  // nothing to zero behind the last row of the band
    const int d0 = 4 * lane;
    const bool inside = d0 >= lo_d && d0 + 3 < hi_e, outside = d0 + 3 < lo_d || d0 >= hi_e;
    const bool act4 = lane < nchunks && (inside || outside);
    const unsigned voff4 = inside ? (unsigned)(16 * lane + iy_start * g.W) : OOB;
    const int q1 = (lo_d & 3) ? (lo_d >> 6) : -1, q2 = (r_hi < g.NR && (hi_d & 3)) ? (hi_d >> 6) : -1;
    auto fix = [&](unsigned *dst, int soff, int q) {
      const int d = 64 * q + lane;
      const bool mine = ((d >> 2) == (lo_d >> 2) && (lo_d & 3)) || ((d >> 2) == (hi_d >> 2) && r_hi < g.NR && (hi_d & 3));
      const unsigned voff = (d >= lo_d && d < hi_d) ? (unsigned)(4 * d + iy_start * g.W) : OOB;
      if (mine) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_in, (lds_ptr_t)(dst + 64 * q), 4, (int)voff, soff, 0, 0);
    };
#pragma unroll 1
    for (int cc = 0; cc < CPW; cc++) {
      const int c = wave + NWV * cc;
      const int soff = ((b * g.CH + c0 + c) * g.H) * g.W;
      unsigned *dst = dw_lds + c * g.CSD;
      if (act4) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_in, (lds_ptr_t)dst, 16, (int)voff4, soff, 0, 0);
      if (q1 >= 0) fix(dst, soff, q1);
      if (q2 >= 0 && q2 != q1) fix(dst, soff, q2);
    }
  } else {
    v4i ld[CPW][2];
    int mis[CPW];
#pragma unroll
    for (int cc = 0; cc < CPW; cc++) {
      const long long pl_ = min((long long)b * g.CH + min(c0 + wave + NWV * cc, g.CH - 1), g.planes - 1);
      const uint8_t *g0 = g.in + (pl_ * g.H + min(max(iy_start + r_lo, 0), g.H - 1)) * g.W;
      mis[cc] = (int)((uintptr_t)g0 & 15);
      const int last = max(((run_len + mis[cc] + 15) >> 4) - 1, 0);
      // lanes past the end of the run re-read its last chunk (masked off below)
      ld[cc][0] = *(const v4i *)(g0 - mis[cc] + 16 * min(lane, last));
      if (two) ld[cc][1] = *(const v4i *)(g0 - mis[cc] + 16 * min(lane + 64, last));
    }
#pragma unroll
    for (int cc = 0; cc < CPW; cc++) {
      const int c = wave + NWV * cc;
      const int dst = c * g.CSD + r_lo * LWD;
      const unsigned keep = (c0 + c < g.CH && (long long)b * g.CH + c0 + c < g.planes) ? 0xFFFFFFFFu : 0u;
#pragma unroll
      for (int t = 0; t < 2; t++) {
        if (t == 1 && !two) break;
        const int o = 16 * (lane + 64 * t) - mis[cc];  // byte offset of this chunk in the run
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const int ob = o + 4 * u;
          const bool ok = ob >= 0 && ob < run_len;
          dw_lds[ok ? dst + (ob >> 2) : dummy] = ((unsigned)ld[cc][t][u] & keep) ^ 0x80808080u;
        }
      }
      // rows of the band above / below the image
      unsigned *base = dw_lds + c * g.CSD;
      for (int q = lane; q < r_lo * LWD; q += 64) base[q] = 0x80808080u;
      for (int q = r_hi * LWD + lane; q < g.NR * LWD; q += 64) base[q] = 0x80808080u;
    }
  }

  // ---- per-lane channel constants ------------------------------------------------
  const bool ch_ok = c0 + lane < g.CH && (long long)b * g.CH + c0 + lane < g.planes;
  const int ch = (c0 + lane) % g.CHR;  // real channel: index of the weights and constants
  unsigned wA[3], wB[3];
  int corr = 0;
  bn_t kk = 0, ll = 0;
  if (ch_ok) {
    int wsum = 0;
#pragma unroll
    for (int i = 0; i < 3; i++) {
      const int8_t *p = g.wt + (long long)ch * 9 + 3 * i;
      const unsigned k0 = (uint8_t)p[0], k1 = (uint8_t)p[1], k2 = (uint8_t)p[2];
      wA[i] = k0 | (k1 << 8) | (k2 << 16);
      wB[i] = wA[i] << 8;
      wsum += (int)p[0] + (int)p[1] + (int)p[2];
    }
    corr = 128 * wsum + (g.bias ? (int)g.bias[ch] : 0);
    if (MODE == EPI_BN) {
      kk = e.k[ch];
      ll = e.lambda[ch];
    }
  } else {
#pragma unroll
    for (int i = 0; i < 3; i++) wA[i] = wB[i] = 0;
  }
  const bool k_small = __all(bn_k_small(kk));
  if constexpr (DMA) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's LDS-direct loads have landed
  __syncthreads();

  // ---- compute -------------------------------------------------------------------------
  const int xgroups = (g.Wo + 3) >> 2;
  const unsigned *lbase = dw_lds + lane * g.CSD - 1;
  DwColumn col;
  col.LWD = LWD;
  col.rows = rows;
  col.row_bytes = (long long)g.Wo * g.CHR;
  col.corr = corr;
  col.k = kk;
  col.lambda = ll;
  col.mult = e.mult;
  col.shift = e.shift;
  col.sel1 = quad_sel1(lane);
  col.sel2 = quad_sel2(lane);
#pragma unroll
  for (int i = 0; i < 3; i++) {
    col.wA[i] = wA[i];
    col.wB[i] = wB[i];
  }
  const int cq = lane & ~3;
  const bool fastq = (MODE == EPI_BN) ? k_small : (e.shift >= 16);
  constexpr int NS = ((4 - PL) + 3 * S + 2) / 4 + 1;

  for (int xg = wave; xg < xgroups; xg += NWV) {
    col.dc0 = xg * S - 1;  // dword column of the first dword of the window
    col.p = lbase + xg * S;
    // this lane stores 4 consecutive channels of one pixel: plane pq .. pq+3 -> image pq / CHR, channel pq % CHR
    const long long pq = (long long)b * g.CH + c0 + cq;
    col.o = g.out + (((pq / g.CHR) * g.Ho + oy0) * g.Wo + 4 * xg + (lane & 3)) * g.CHR + (int)(pq % g.CHR);
    // 0: store a dword, 1: store the valid bytes one by one, 2: nothing to store
    const long long left = min((long long)(g.CH - c0 - cq), g.planes - pq);  // planes this lane may write
    col.store = (4 * xg + (lane & 3) >= g.Wo || left <= 0) ? 2 : ((g.out_vec4 && left >= 4) ? 0 : 1);
    col.nbytes = (int)min(4ll, max(left, 0ll));
    const bool edge = col.dc0 < 0 || col.dc0 + NS > LWD;
    if (fastq) {
      if (edge) dw3x3_column<S, PL, MODE, FULL, true, true, DMA>(col);
      else dw3x3_column<S, PL, MODE, FULL, false, true, DMA>(col);
    } else {
      if (edge) dw3x3_column<S, PL, MODE, FULL, true, false, DMA>(col);
      else dw3x3_column<S, PL, MODE, FULL, false, false, DMA>(col);
    }
  }
}

#define DW_REG_WAVES 4  // waves per workgroup of the register-resident kernels (independent of each other)

// 3x3 depthwise on small square planes (8x8 or 4x4 input, padding 1): a lane keeps the whole
// plane of its channel in registers (64 or 16 bytes, 16-byte loads; the planes of consecutive
// channels are contiguous in a CHW image, so a wave reads one contiguous 4 KB / 1 KB run) and
// works through all its output pixels with the same v_dot4 windows, requantisation and quad
// transpose as dw3x3_column.  No LDS, no barrier, waves independent: such a layer is a few
// MB at batch 256, and with the staged kernel its time goes into the latency chain load ->
// LDS -> barrier -> arithmetic of a thousand eight-wave workgroups, only part of which are
// resident at a time.
// A filter row that falls outside the plane contributes -128 * (sum of its weights) to every
// output (activations are held as a - 128, and a = 0 there), added as one constant.
// HWC: the input is HWC (the layout glue fused in): a lane quad loads a dword (its four channels)
// of four neighbouring pixels each and transposes it into four pixels of each lane's channel.
template <int HW, int S, int MODE, bool HWC>
__global__ __launch_bounds__(64 * DW_REG_WAVES) void dw3x3_plane_kernel(DwGeom g, EpiArgs e)
{
  constexpr int RD = HW / 4;                  // dwords per row
  constexpr int HO = (HW - 1) / S + 1;        // output rows and columns
  constexpr int XG = HO / 4;                  // groups of 4 output columns
  constexpr int O0 = 3;                       // byte offset of column -1 in a span that starts one dword left of the group
  constexpr int NS = (O0 + 3 * S + 2) / 4 + 1;
  static_assert(HW % 4 == 0 && HO % 4 == 0, "whole dwords in, whole groups of 4 columns out");
  // the waves of a workgroup are independent work items (fewer, larger workgroups start sooner:
  // this kernel lasts a few microseconds)
  const int lane = threadIdx.x & 63;
  const long long item = (long long)blockIdx.x * DW_REG_WAVES + (threadIdx.x >> 6);
  if (item >= (long long)g.B * g.cgroups) return;
  const int cg = (int)(item % g.cgroups), b = (int)(item / g.cgroups);
  const int ch = cg * DW_CG + lane;           // CH % 64 == 0

  const unsigned sel1 = quad_sel1(lane), sel2 = quad_sel2(lane);
  unsigned row[HW][RD];
  if constexpr (HWC) {
    const uint8_t *src = g.in + ((long long)b * (HW * HW) + (lane & 3)) * g.CH + (ch & ~3);
#pragma unroll
    for (int y = 0; y < HW; y++)
#pragma unroll
      for (int d = 0; d < RD; d++) row[y][d] = *(const unsigned *)(src + (long long)(y * HW + 4 * d) * g.CH);
#pragma unroll
    for (int y = 0; y < HW; y++)
#pragma unroll
      for (int d = 0; d < RD; d++) row[y][d] = quad_transpose4x4_perm(row[y][d], sel1, sel2) ^ 0x80808080u;
  } else {
    const uint8_t *src = g.in + ((long long)b * g.CH + ch) * (HW * HW);
#pragma unroll
    for (int q = 0; q < HW * RD / 4; q++) {
      const v4i v = *(const v4i *)(src + 16 * q);
#pragma unroll
      for (int j = 0; j < 4; j++) row[(4 * q + j) / RD][(4 * q + j) % RD] = (unsigned)v[j] ^ 0x80808080u;
    }
  }
  unsigned wA[3], wB[3];
  int pad[3], wsum = 0;
#pragma unroll
  for (int i = 0; i < 3; i++) {
    const int8_t *p = g.wt + (long long)ch * 9 + 3 * i;
    const unsigned k0 = (uint8_t)p[0], k1 = (uint8_t)p[1], k2 = (uint8_t)p[2];
    wA[i] = k0 | (k1 << 8) | (k2 << 16);
    wB[i] = wA[i] << 8;
    const int rs = (int)p[0] + (int)p[1] + (int)p[2];
    pad[i] = -128 * rs;
    wsum += rs;
  }
  const int corr = 128 * wsum + (g.bias ? (int)g.bias[ch] : 0);
  bn_t kk = 0, ll = 0;
  if (MODE == EPI_BN) {
    kk = e.k[ch];
    ll = e.lambda[ch];
  }
  const bool fastq = (MODE == EPI_BN) ? __all(bn_k_small(kk)) : (e.shift >= 16);
  // after the quad transpose this lane holds 4 consecutive channels of pixel column 4*xg + lane%4
  uint8_t *obase = g.out + ((long long)b * HO * HO + (lane & 3)) * g.CH + cg * DW_CG + (lane & ~3);

  auto body = [&](auto fq) {
    constexpr bool FASTQ = decltype(fq)::value;
#pragma unroll
    for (int oy = 0; oy < HO; oy++) {
#pragma unroll
      for (int xg = 0; xg < XG; xg++) {
        int acc[4] = {corr, corr, corr, corr};
#pragma unroll
        for (int i = 0; i < 3; i++) {
          const int iy = oy * S - 1 + i;
          if (iy < 0 || iy >= HW) {
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] += pad[i];
          } else {
            unsigned span[NS];
#pragma unroll
            for (int d = 0; d < NS; d++) {
              const int col = xg * S - 1 + d;  // dword column
              span[d] = (col >= 0 && col < RD) ? row[iy][col < 0 ? 0 : (col >= RD ? RD - 1 : col)] : 0x80808080u;
            }
            dw_tap<O0, NS>(span, wA[i], wB[i], acc[0]);
            dw_tap<O0 + S, NS>(span, wA[i], wB[i], acc[1]);
            dw_tap<O0 + 2 * S, NS>(span, wA[i], wB[i], acc[2]);
            dw_tap<O0 + 3 * S, NS>(span, wA[i], wB[i], acc[3]);
          }
        }
        unsigned packed = requant4_same<MODE, FASTQ>(acc[0], acc[1], acc[2], acc[3], kk, ll, e.mult, e.shift);
        packed = quad_transpose4x4_perm(packed, sel1, sel2);
        *(unsigned *)(obase + (long long)(oy * HO + 4 * xg) * g.CH) = packed;
      }
    }
  };
  if (fastq) body(std::true_type{});
  else body(std::false_type{});
}

// The same for planes with rows of 16, 32 or 64 bytes (padding 1): a lane keeps the (R-1)*S + 3
// input rows behind R output rows of its plane in registers, a workgroup (one wave) takes 64
// consecutive planes of the batch (B * CH planes lie back to back; CH % 4 == 0 keeps the four
// channels that a lane quad transposes inside one image) and one segment of R output rows.
// Rows above and below the plane are loaded from a valid address and replaced by zero
// activations.
template <int WB, int R, int S, int MODE, bool HWC>
__global__ __launch_bounds__(64 * DW_REG_WAVES) void dw3x3_rows_kernel(DwGeom g, EpiArgs e)
{
  constexpr int RD = WB / 4;                  // dwords per row
  constexpr int WO = (WB - 1) / S + 1;        // output columns
  constexpr int XG = WO / 4;                  // groups of 4 output columns
  constexpr int NIN = (R - 1) * S + 3;        // input rows behind R output rows
  constexpr int O0 = 3;
  constexpr int NS = (O0 + 3 * S + 2) / 4 + 1;
  static_assert(WB % 16 == 0 && WO % 4 == 0, "whole 16-byte pieces in, whole groups of 4 columns out");
  const int lane = threadIdx.x & 63;
  const int nseg = (g.Ho + R - 1) / R;
  const long long item = (long long)blockIdx.x * DW_REG_WAVES + (threadIdx.x >> 6);  // one per wave
  if (item >= g.planes / DW_CG * nseg) return;
  const int seg = (int)(item % nseg);
  const long long P = item / nseg * DW_CG + lane;  // plane: image P / CHR, channel P % CHR
  const int b = (int)(P / g.CHR), ch = (int)(P % g.CHR);
  const int oy0 = seg * R;

  const unsigned sel1 = quad_sel1(lane), sel2 = quad_sel2(lane);
  unsigned row[NIN][RD];
  if constexpr (HWC) {
    const uint8_t *src = g.in + ((long long)b * g.H * WB + (lane & 3)) * g.CHR + (ch & ~3);
#pragma unroll
    for (int r = 0; r < NIN; r++) {
      const int iy = oy0 * S - 1 + r;
      const bool ok = (unsigned)iy < (unsigned)g.H;
      const uint8_t *rp = src + (long long)min(max(iy, 0), g.H - 1) * WB * g.CHR;
#pragma unroll
      for (int d = 0; d < RD; d++) {
        const unsigned v = *(const unsigned *)(rp + (long long)(4 * d) * g.CHR);
        row[r][d] = ok ? v : 0u;
      }
    }
#pragma unroll
    for (int r = 0; r < NIN; r++)
#pragma unroll
      for (int d = 0; d < RD; d++) row[r][d] = quad_transpose4x4_perm(row[r][d], sel1, sel2) ^ 0x80808080u;
  } else {
    const uint8_t *src = g.in + P * ((long long)g.H * WB);
#pragma unroll
    for (int r = 0; r < NIN; r++) {
      const int iy = oy0 * S - 1 + r;
      const bool ok = (unsigned)iy < (unsigned)g.H;
      const uint8_t *rp = src + (long long)min(max(iy, 0), g.H - 1) * WB;
#pragma unroll
      for (int q = 0; q < RD / 4; q++) {
        const v4i v = *(const v4i *)(rp + 16 * q);
#pragma unroll
        for (int j = 0; j < 4; j++) row[r][4 * q + j] = (ok ? (unsigned)v[j] : 0u) ^ 0x80808080u;
      }
    }
  }
  unsigned wA[3], wB[3];
  int wsum = 0;
#pragma unroll
  for (int i = 0; i < 3; i++) {
    const int8_t *p = g.wt + (long long)ch * 9 + 3 * i;
    const unsigned k0 = (uint8_t)p[0], k1 = (uint8_t)p[1], k2 = (uint8_t)p[2];
    wA[i] = k0 | (k1 << 8) | (k2 << 16);
    wB[i] = wA[i] << 8;
    wsum += (int)p[0] + (int)p[1] + (int)p[2];
  }
  const int corr = 128 * wsum + (g.bias ? (int)g.bias[ch] : 0);
  bn_t kk = 0, ll = 0;
  if (MODE == EPI_BN) {
    kk = e.k[ch];
    ll = e.lambda[ch];
  }
  const bool fastq = (MODE == EPI_BN) ? __all(bn_k_small(kk)) : (e.shift >= 16);
  // after the quad transpose this lane holds the 4 channels of its quad for pixel column 4*xg + lane%4
  uint8_t *obase = g.out + (((long long)b * g.Ho + oy0) * WO + (lane & 3)) * g.CHR + (ch & ~3);

  auto body = [&](auto fq) {
    constexpr bool FASTQ = decltype(fq)::value;
#pragma unroll
    for (int ro = 0; ro < R; ro++) {
      if (oy0 + ro >= g.Ho) break;  // (the same for all lanes)
#pragma unroll
      for (int xg = 0; xg < XG; xg++) {
        int acc[4] = {corr, corr, corr, corr};
#pragma unroll
        for (int i = 0; i < 3; i++) {
          unsigned span[NS];
#pragma unroll
          for (int d = 0; d < NS; d++) {
            const int col = xg * S - 1 + d;  // dword column
            span[d] = (col >= 0 && col < RD) ? row[ro * S + i][col < 0 ? 0 : (col >= RD ? RD - 1 : col)] : 0x80808080u;
          }
          dw_tap<O0, NS>(span, wA[i], wB[i], acc[0]);
          dw_tap<O0 + S, NS>(span, wA[i], wB[i], acc[1]);
          dw_tap<O0 + 2 * S, NS>(span, wA[i], wB[i], acc[2]);
          dw_tap<O0 + 3 * S, NS>(span, wA[i], wB[i], acc[3]);
        }
        unsigned packed = requant4_same<MODE, FASTQ>(acc[0], acc[1], acc[2], acc[3], kk, ll, e.mult, e.shift);
        packed = quad_transpose4x4_perm(packed, sel1, sel2);
        *(unsigned *)(obase + (long long)(ro * WO + 4 * xg) * g.CHR) = packed;
      }
    }
  };
  if (fastq) body(std::true_type{});
  else body(std::false_type{});
}

// Any kernel size / stride / padding: one output per lane per step, one LDS
// byte read per tap.  Weights are read through L1 (lane stride ky*kx bytes).
template <int MODE>
__global__ __launch_bounds__(256) void dw_generic_kernel(DwGeom g, EpiArgs e)
{
  extern __shared__ unsigned dw_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  int id = dw_xcd_remap(blockIdx.x, g.total);
  const int cg = id % g.cgroups;
  id /= g.cgroups;
  const int band = id % g.bands;
  const int b = id / g.bands;
  const int c0 = cg * DW_CG;
  const int oy0 = band * g.RB;
  const int rows = min(g.RB, g.Ho - oy0);

  const uint8_t *img = g.in + (long long)b * g.CH * g.H * g.W;
  dw_stage(g, dw_lds, img, c0, oy0 * g.sy - g.pt);

  const int ch = c0 + lane;
  const bool ch_ok = ch < g.CH;
  const int taps = g.kx * g.ky;
  const int8_t *wp = g.wt + (long long)(ch_ok ? ch : 0) * taps;
  int corr = 0;
  bn_t kk = 0, ll = 0;
  if (ch_ok) {
    int wsum = 0;
    for (int t = 0; t < taps; t++) wsum += (int)wp[t];
    corr = 128 * wsum + (g.bias ? (int)g.bias[ch] : 0);
    if (MODE == EPI_BN) {
      kk = e.k[ch];
      ll = e.lambda[ch];
    }
  }
  __syncthreads();

  const int8_t *lb = (const int8_t *)(dw_lds + lane * g.CSD) + (g.LP - g.pl);
  const int rowbytes = g.LWD * 4;
  uint8_t *obase = g.out + (((long long)b * g.Ho + oy0) * g.Wo) * g.CH + ch;
  const int items = rows * g.Wo;
  for (int it = wave; it < items; it += 4) {
    const int r = it / g.Wo, ox = it - r * g.Wo;
    int acc = corr;
    const int8_t *p = lb + (r * g.sy) * rowbytes + ox * g.sx;
    for (int fy = 0; fy < g.ky; fy++)
      for (int fx = 0; fx < g.kx; fx++)
        acc += (int)p[fy * rowbytes + fx] * (int)wp[fy * g.kx + fx];
    if (ch_ok) obase[((long long)r * g.Wo + ox) * g.CH] = (uint8_t)requant<MODE>(acc, kk, ll, e.mult, e.shift);
  }
}

// HWC -> CHW layout change with optional zero rows above and below each plane:
// the glue between a conv / pointwise output and a depthwise input (the
// reference leaves this step to the application).  out is [C][pad_t+H+pad_b][W].
__global__ __launch_bounds__(256) void hwc_to_chw_kernel(const uint8_t *in, uint8_t *out, int H, int W, int C,
                                                         int pad_t, int pad_b, int tiles_p, int tiles_c)
{
  // tile: 64 pixels x 64 channels through LDS
  __shared__ uint8_t tile[64][65];
  int id = blockIdx.x;
  const int tc = id % tiles_c;
  id /= tiles_c;
  const int tp = id % tiles_p;
  const int b = id / tiles_p;
  const int HW = H * W;
  const int Hp = pad_t + H + pad_b;
  const uint8_t *src = in + (long long)b * HW * C;
  uint8_t *dst = out + (long long)b * C * Hp * W;
  const int p0 = tp * 64, c0 = tc * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int p = p0 + i, c = c0 + tx;
    tile[i][tx] = (p < HW && c < C) ? src[(long long)p * C + c] : 0;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int c = c0 + i, p = p0 + tx;
    if (c < C && p < HW) dst[((long long)c * Hp + pad_t) * W + p] = tile[tx][i];
  }
  // zero rows
  if (tp == 0 && (pad_t | pad_b)) {
    for (int i = ty; i < 64; i += 4) {
      const int c = c0 + i;
      if (c >= C) continue;
      for (int x = tx; x < pad_t * W; x += 64) dst[(long long)c * Hp * W + x] = 0;
      for (int x = tx; x < pad_b * W; x += 64) dst[((long long)c * Hp + pad_t + H) * W + x] = 0;
    }
  }
}

// 4x4 byte transpose inside one lane: r[i] = bytes of pixel i (4 channels) ->
// t[j] = bytes of channel j (4 pixels).
__device__ __forceinline__ void transpose4x4_bytes(const unsigned (&r)[4], unsigned (&t)[4])
{
  // __builtin_amdgcn_perm(hi, lo, sel): selector 0-3 picks bytes of lo, 4-7 bytes of hi
  const unsigned a0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400);  // p0c0 p1c0 p0c1 p1c1
  const unsigned a1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602);  // p0c2 p1c2 p0c3 p1c3
  const unsigned b0 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400);  // p2c0 p3c0 p2c1 p3c1
  const unsigned b1 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602);
  t[0] = __builtin_amdgcn_perm(b0, a0, 0x05040100);
  t[1] = __builtin_amdgcn_perm(b0, a0, 0x07060302);
  t[2] = __builtin_amdgcn_perm(b1, a1, 0x05040100);
  t[3] = __builtin_amdgcn_perm(b1, a1, 0x07060302);
}

// Fast HWC -> CHW for C % 16 == 0, H*W % 4 == 0 and 16-byte aligned maps: a tile of
// 256 pixels x 64 channels goes through LDS; reads are 16 bytes per lane (64 contiguous
// bytes per pixel), writes are one dword of 4 pixels per lane, 256 contiguous bytes per
// channel and store instruction.
template <bool NT>
__global__ __launch_bounds__(256) void hwc_to_chw_fast_kernel(const uint8_t *in, uint8_t *out, int H, int W, int C,
                                                              int pad_t, int pad_b, int tiles_p, int tiles_c)
{
  constexpr int P = 80;  // LDS row pitch in bytes (16-byte aligned rows)
  __shared__ __attribute__((aligned(16))) uint8_t tile[256 * P];
  int id = blockIdx.x;
  const int tc = id % tiles_c;
  id /= tiles_c;
  const int tp = id % tiles_p;
  const int b = id / tiles_p;
  const int HW = H * W;
  const int Hp = pad_t + H + pad_b;
  const uint8_t *src = in + (long long)b * HW * C;
  uint8_t *dst = out + (long long)b * C * Hp * W;
  const int p0 = tp * 256, c0 = tc * 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  {
    const int chunk = tid & 3, c = c0 + 16 * chunk;
    v4i v[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int p = min(p0 + (tid >> 2) + 64 * i, HW - 1);
      v[i] = *(const v4i *)(src + (long long)p * C + min(c, C - 16));
    }
#pragma unroll
    for (int i = 0; i < 4; i++) *(v4i *)&tile[((tid >> 2) + 64 * i) * P + 16 * chunk] = v[i];
  }
  __syncthreads();
  const int cw = c0 + 16 * wave;  // this wave's 16 channels
  const int p = p0 + 4 * lane;    // this lane's 4 pixels
  if (cw < C && p < HW) {
    unsigned rows[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const v4i r = *(const v4i *)&tile[(4 * lane + i) * P + 16 * wave];
      rows[i][0] = (unsigned)r.x;
      rows[i][1] = (unsigned)r.y;
      rows[i][2] = (unsigned)r.z;
      rows[i][3] = (unsigned)r.w;
    }
    uint8_t *o = dst + ((long long)cw * Hp + pad_t) * W + p;
    const long long plane = (long long)Hp * W;
#pragma unroll
    for (int d = 0; d < 4; d++) {
      const unsigned r[4] = {rows[0][d], rows[1][d], rows[2][d], rows[3][d]};
      unsigned t[4];
      transpose4x4_bytes(r, t);
#pragma unroll
      for (int j = 0; j < 4; j++) store4<NT>(o + (4 * d + j) * plane, (int)t[j]);
    }
  }
  // zero rows
  if (tp == 0 && (pad_t | pad_b)) {
    for (int i = wave; i < 64; i += 4) {
      const int c = c0 + i;
      if (c >= C) continue;
      for (int x = lane; x < pad_t * W; x += 64) dst[(long long)c * Hp * W + x] = 0;
      for (int x = lane; x < pad_b * W; x += 64) dst[((long long)c * Hp + pad_t + H) * W + x] = 0;
    }
  }
}
