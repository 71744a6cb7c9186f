// Implicit-GEMM kernel for standard / pointwise convolution and linear layers.
//
// Replaces the reference's per-core im2col + 4x2 SumDotp matmul
// (32bit/src/pulp_nn_conv_Ho_parallel.c:76-183, pulp_nn_matmul.c:53-216,
// pulp_nn_pointwise_HoWo_parallel.c:97-120, pulp_nn_linear.c:58-108) by one
// kernel: GEMM with M = batch*Ho*Wo pixels, N = output channels,
// K = ky*kx*Ci taken in the (ky, kx, ci) order of an OHWI weight row.
//
// CDNA4 mapping
//   * v_mfma_i32_16x16x64_i8: weights are the row operand, pixels the column
//     operand, so that one lane ends up with 4*TN consecutive output channels
//     of one pixel (one vector store into the HWC output).
//   * The MFMA multiplies signed bytes but activations are unsigned.  They are
//     staged as a ^ 0x80 (= a - 128 as int8) and 128 * sum_k w[n][k] is added
//     back per output channel; taps that fall outside the image (a = 0) are
//     staged as 0x80.  The weight sums are accumulated with v_dot4 from the
//     weight bytes as they pass through registers on their way to LDS, so no
//     extra pass over the weights and no extra launch is needed.  All of it is
//     exact in wrapping 32-bit arithmetic.
//   * Tiles of BM pixels x 64 bytes of K and BN channels x 64 bytes of K are
//     double-buffered in LDS with a 16-byte-chunk XOR swizzle so that both the
//     staging writes and the ds_read_b128 fragment reads are conflict free.
//   * The im2col gather is never materialised: each 16-byte chunk of a K slice
//     is one coalesced global load from the HWC input (GATHER_CHUNK16, needs
//     Ci % 16 == 0), or a byte gather for any other geometry (GATHER_BYTES).
//     With Ci % 64 == 0 (GATHER_UNIFORM) a whole K slice lies inside one filter tap, so
//     the tap walk is scalar work shared by the wave, and the loads are buffer loads whose
//     hardware range check supplies the zeros: a pixel's offset is fixed for the whole
//     kernel, the tap adds a scalar offset, and an out-of-image tap (one bit per tap and
//     pixel, computed once) ORs the offset to 0xffffffff, which the range check turns
//     into a load of zeros.  Per K slice that is two VALU instructions per 16-byte chunk
//     of activations and none per chunk of weights.
//     With 16 or 32 input channels (GATHER_SUBTAP) a K slice holds four or two whole taps: the
//     same buffer loads, with the tap of a lane's chunk fixed relative to the slice, so the tap
//     offset is a handful of VALU instructions per load instead of the general per-chunk
//     arithmetic (divisions, bounds checks, 64-bit addresses), which is what such small layers
//     otherwise spend their time on.
#pragma once
#include <type_traits>

#include "memops.h"
#include "requant.h"

enum { GATHER_CHUNK16 = 0, GATHER_BYTES = 1, GATHER_UNIFORM = 2, GATHER_SUBTAP = 3 };
enum { EPI_OUT32 = 3 };  // linear_out_32: int32 accumulators + int32 bias, no requantisation

// Division of a 32-bit unsigned number by a divisor fixed for the launch, as a multiply-high, an add and
// two shifts (Granlund & Montgomery); the host computes the constants.  The compiler's expansion of a
// 32-bit division is some 40 instructions, and a tile's set-up divides several times per lane.
struct FastDiv {
  unsigned mul, sh1, sh2;
};
static inline FastDiv fastdiv_make(unsigned d)
{
  FastDiv f;
  unsigned l = 0;
  while ((1ull << l) < d) l++;  // ceil(log2(d))
  f.mul = (unsigned)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
  f.sh1 = l < 1 ? l : 1;
  f.sh2 = l > 1 ? l - 1 : 0;
  return f;
}
__device__ __forceinline__ unsigned fastdiv(unsigned n, const FastDiv &f)
{
  const unsigned t = __umulhi(n, f.mul);
  return (t + ((n - t) >> f.sh1)) >> f.sh2;
}

struct ConvGeom {
  const uint8_t *in;
  const int8_t *w;
  const int8_t *bias;  // int8 [N]; int32 [N] for EPI_OUT32; may be null
  void *out;
  int M, N, K;
  int H, W, Ci;
  int Ho, Wo, HoWo;
  int kx, ky;
  int pt, pl, sx, sy;
  long long in_img;    // bytes per input image
  int vec_store;       // output rows may be written with 4*TN-byte vector stores
  int nt;              // write the output with non-temporal stores
  int tiles_n;         // number of channel tiles
  int tiles_total;     // tiles_m * tiles_n
  FastDiv d_howo, d_wo, d_tiles_n;  // divisions by HoWo, Wo, tiles_n
  int batch;           // number of images: ceil(M / HoWo)
  int ci_shift;        // log2(Ci) when Ci is a power of two (GATHER_SUBTAP), else 0
  int rkx;             // 65536 / kx + 1: t * rkx >> 16 == t / kx for t < 32 (GATHER_SUBTAP)
  int cpt;             // Ci / 64: K sub-slices per filter tap (igemm_ring_kernel)
  FastDiv d_cpt, d_kx; // divisions by cpt and kx (igemm_ring_kernel)
  int rgroups;         // groups of 4 output rows per image (igemm_patch_kernel)
  FastDiv d_rg;        // division by rgroups
};

#define IGEMM_BK 64
#ifndef IGEMM_MINB
#define IGEMM_MINB 3  // workgroups per CU the register budget is sized for
#endif

// Tile index of this workgroup.  Workgroups are dealt round-robin to the 8
// XCDs; the remap gives each XCD a contiguous range of tiles so that tiles
// sharing input pixels (same tile_m) and neighbouring rows hit the same L2.
__device__ __forceinline__ int xcd_remap(int id, int total)
{
  const int q = total >> 3, rem = total & 7;
  const int x = id & 7, s = id >> 3;
  return x * q + min(x, rem) + s;
}

__device__ __forceinline__ int lds_off(int row, int chunk)
{
  return row * IGEMM_BK + ((chunk ^ ((row >> 1) & 3)) << 4);
}

// Epilogue shared by the tiled kernels.  acc[t][s][r] = channel cb + 4*t + r of pixel
// m0 + wm0 + 16*s + l16, where cb = wn0 + (lane/16)*4*TN; wm0 / wn0: offset of the wave's tile inside
// the workgroup tile.  wsum is indexed by LDS weight row, cbias / ck_ / cl_ by channel inside the tile.
// Channel constants are fetched four channels (one MFMA tile row group) at a time to
// keep the register footprint of the epilogue below that of the main loop.
template <int TN, int TM, int MODE>
__device__ __forceinline__ void igemm_epilogue(v4i (&acc)[TN][TM], const ConvGeom &g, const EpiArgs &e, int m0, int n0,
                                               int wm0, int wn0, int lane, const int *wsum, const int *cbias,
                                               const bn_t *ck_, const bn_t *cl_)
{
  const int l16 = lane & 15, lgrp = lane >> 4;
  const int cb = wn0 + lgrp * (4 * TN);
  const bool acc24 = g.K <= 256;  // |acc| <= K * 255 * 128 + 128 < 2^23
  constexpr int QM = MODE == EPI_OUT32 ? EPI_RAW : MODE;
  unsigned packed[TM][TN];
#pragma unroll
  for (int t = 0; t < TN; t++) {
    int corr[4];
    bn_t kk[4], ll[4];
    bool ks = true;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int c = cb + 4 * t + r;  // channel inside the tile (constants of channels past N are zero)
      kk[r] = (MODE == EPI_BN) ? ck_[c] : (bn_t)0;
      ll[r] = (MODE == EPI_BN) ? cl_[c] : (bn_t)0;
      ks = ks && bn_k_small(kk[r]);
      corr[r] = cbias[c] + 128 * wsum[wn0 + 16 * t + 4 * lgrp + r];
    }
    const bool k_small = __all(ks);  // wave-uniform precondition of the fast batch-norm form
#pragma unroll
    for (int s = 0; s < TM; s++) {
      const int a0 = acc[t][s][0] + corr[0], a1 = acc[t][s][1] + corr[1];
      const int a2 = acc[t][s][2] + corr[2], a3 = acc[t][s][3] + corr[3];
      if constexpr (MODE == EPI_OUT32) {
        const int m = m0 + wm0 + 16 * s + l16;
        if (m < g.M) {
          int *o = (int *)g.out + (long long)m * g.N + n0 + cb + 4 * t;
          const int v[4] = {a0, a1, a2, a3};
#pragma unroll
          for (int r = 0; r < 4; r++)
            if (n0 + cb + 4 * t + r < g.N) o[r] = v[r];
        }
      } else {
        packed[s][t] = acc24 ? requant4<QM, true>(a0, a1, a2, a3, kk, ll, k_small, e.mult, e.shift)
                             : requant4<QM, false>(a0, a1, a2, a3, kk, ll, k_small, e.mult, e.shift);
      }
    }
  }
  if constexpr (MODE != EPI_OUT32) {
    // one copy of the store code per cache policy
    auto put = [&](auto nt) {
      constexpr bool NT = decltype(nt)::value;
#pragma unroll
      for (int s = 0; s < TM; s++) {
        const int m = m0 + wm0 + 16 * s + l16;
        if (m >= g.M) continue;
        uint8_t *o = (uint8_t *)g.out + (long long)m * g.N + n0 + cb;
        if (g.vec_store && n0 + cb + 4 * TN <= g.N) {
          if constexpr (TN == 4) store16<NT>(o, (v4i){(int)packed[s][0], (int)packed[s][1 % TN], (int)packed[s][2 % TN], (int)packed[s][3 % TN]});
          else if constexpr (TN == 2) store8<NT>(o, (v2i){(int)packed[s][0], (int)packed[s][1 % TN]});
          else store4<NT>(o, (int)packed[s][0]);
        } else {
#pragma unroll
          for (int c = 0; c < 4 * TN; c++)
            if (n0 + cb + c < g.N) o[c] = (uint8_t)(packed[s][c >> 2] >> (8 * (c & 3)));
        }
      }
    };
    if (g.nt) put(std::true_type{});
    else put(std::false_type{});
  }
}

// ONEPASS > 0: the layer has at most ONEPASS K slices and the whole K extent of a tile is staged at
// once: all global loads of the tile are issued back to back (one memory round trip instead of one
// per slice), then staged, and after a single barrier the slices are multiplied one after the other.
// Layers this short are bound by those round trips, not by bytes or multiplies.
template <int TN, int WAVES_M, int WAVES_N, int GATHER, int MODE, int TM = 4, int ONEPASS = 0>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N,
                            (WAVES_M * WAVES_N > 8 || TM > 4) ? 1 : (WAVES_M * WAVES_N > 4 || GATHER == GATHER_BYTES || ONEPASS ? 2 : IGEMM_MINB))
void igemm_kernel(ConvGeom g, EpiArgs e)
{
  constexpr int NBUF = ONEPASS ? ONEPASS : 2;  // K slices resident in LDS
  constexpr int WM = 16 * TM, WN = 16 * TN;
  constexpr int BM = WM * WAVES_M, BN = WN * WAVES_N;
  constexpr int NTH = 64 * WAVES_M * WAVES_N;    // threads per workgroup
  constexpr int RPP = NTH / 4;                   // tile rows staged per pass (4 threads per 64-byte row)
  constexpr int RA = BM / RPP;                   // activation chunks per thread per K slice
  constexpr int RW = (BN * 4 + NTH - 1) / NTH;   // weight chunks per thread per K slice
  static_assert(BM % RPP == 0, "pixel tile is a whole number of staging passes");

  constexpr bool SUB = GATHER == GATHER_SUBTAP;                  // several taps per K slice
  constexpr bool UNI = GATHER == GATHER_UNIFORM || SUB;          // buffer loads with a fixed offset per pixel
  __shared__ __attribute__((aligned(16))) uint8_t As[NBUF][BM * IGEMM_BK];
  __shared__ __attribute__((aligned(16))) int8_t Ws[NBUF][BN * IGEMM_BK];
  __shared__ int wsum[BN];
  // per-channel constants of the tile, fetched while the first K slice is on its way
  __shared__ int cbias[BN];
  __shared__ bn_t ck_[MODE == EPI_BN ? BN : 1], cl_[MODE == EPI_BN ? BN : 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wave_m = wave % WAVES_M, wave_n = wave / WAVES_M;

  const int tile = xcd_remap(blockIdx.x, g.tiles_total);
  const int tile_m = (int)fastdiv((unsigned)tile, g.d_tiles_n);
  const int m0 = tile_m * BM;
  const int n0 = (tile - tile_m * g.tiles_n) * BN;

  // ---- per-thread gather state -------------------------------------------
  const int ck = tid & 3;  // which 16-byte chunk of the 64-byte K slice
  int iy0[RA], ix0[RA];
  long long abase[RA];
#pragma unroll
  for (int i = 0; i < RA; i++) {
    const int m = m0 + (tid >> 2) + RPP * i;
    if (m < g.M) {
      const int b = (int)fastdiv((unsigned)m, g.d_howo), rem = m - b * g.HoWo;
      const int oy = (int)fastdiv((unsigned)rem, g.d_wo), ox = rem - oy * g.Wo;
      iy0[i] = oy * g.sy - g.pt;
      ix0[i] = ox * g.sx - g.pl;
      abase[i] = (long long)b * g.in_img;
    } else {
      iy0[i] = -(1 << 28);
      ix0[i] = 0;
      abase[i] = 0;
    }
  }
  // GATHER_UNIFORM state.  The activation buffer starts (pt*W + pl)*Ci bytes before the
  // input so that pixel offsets are non-negative; the weight buffer ends after row N-1,
  // so rows past the last channel read as zeros.
  [[maybe_unused]] __amdgpu_buffer_rsrc_t rsrc_a, rsrc_w;
  [[maybe_unused]] unsigned poff[RA], pinv[RA], woff[RW];
  [[maybe_unused]] int u_tap = 0, u_fx = 0, u_fy = 0, u_ci = 0, u_slice = 0;
  if constexpr (UNI) {
    const unsigned shift = (unsigned)((g.pt * g.W + g.pl) * g.Ci);
    const unsigned batch = (unsigned)g.batch;
    rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void *)(g.in - shift), 0, shift + batch * (unsigned)g.in_img, 0x00020000);
    rsrc_w = __builtin_amdgcn_make_buffer_rsrc((void *)g.w, 0, (unsigned)g.N * (unsigned)g.K, 0x00020000);
#pragma unroll
    for (int i = 0; i < RA; i++) {
      const int m = m0 + (tid >> 2) + RPP * i;
      poff[i] = 0xffffffffu;
      pinv[i] = 0;
      if (m < g.M) {
        const int b = (int)fastdiv((unsigned)m, g.d_howo), rem = m - b * g.HoWo;
        const int oy = (int)fastdiv((unsigned)rem, g.d_wo), ox = rem - oy * g.Wo;
        poff[i] = (unsigned)b * (unsigned)g.in_img + (unsigned)((oy * g.sy * g.W + ox * g.sx) * g.Ci) +
                  (SUB ? (16u * ck) & (unsigned)(g.Ci - 1) : 16u * ck);
        if (SUB) pinv[i] = ~0u << (g.kx * g.ky);  // taps past the filter (the tail of the last K slice)
        for (int fy_ = 0, t = 0; fy_ < g.ky; fy_++)
          for (int fx_ = 0; fx_ < g.kx; fx_++, t++) {
            const int iy = oy * g.sy - g.pt + fy_, ix = ox * g.sx - g.pl + fx_;
            if ((unsigned)iy >= (unsigned)g.H || (unsigned)ix >= (unsigned)g.W) pinv[i] |= 1u << t;
          }
      }
    }
  }
  // GATHER_SUBTAP: which of the slice's taps this lane's chunk belongs to, and 65536 / kx rounded up
  // (t * that >> 16 == t / kx for the tap numbers that occur: t < 32, kx <= 32)
  [[maybe_unused]] const int sub_h = SUB ? (16 * ck) >> g.ci_shift : 0;
  [[maybe_unused]] const int sub_rkx = g.rkx;
  // (fy, fx, ci) of byte k = 16*ck of the current K slice
  int kpos = 16 * ck;
  int ci = 0, tap = 0, fy = 0, fx = 0;
  if constexpr (!UNI) {
    ci = kpos % g.Ci, tap = kpos / g.Ci;
    fy = tap / g.kx, fx = tap - fy * g.kx;
  }

  // Weight rows sit in LDS in fragment order: LDS row p = wn*WN + 16*t + i holds
  // channel wn*WN + (i/4)*4*TN + 4*t + (i%4), so that MFMA tile t of a wave reads
  // 16 consecutive LDS rows and each lane ends up with 4*TN consecutive channels.
  int wrow[RW];   // LDS row
  int wchan[RW];  // channel offset inside the tile that this row holds
  bool wact[RW];
  int wpart[RW];
#pragma unroll
  for (int i = 0; i < RW; i++) {
    const int q = tid + NTH * i;
    const int p = q >> 2;
    wrow[i] = p;
    const int pp = p % WN, t = pp >> 4, r16 = pp & 15;
    wchan[i] = (p / WN) * WN + (r16 >> 2) * (4 * TN) + 4 * t + (r16 & 3);
    wact[i] = q < BN * 4;
    wpart[i] = 0;
    if constexpr (UNI) {
      const int n = n0 + wchan[i];
      woff[i] = (wact[i] && n < g.N) ? (unsigned)n * (unsigned)g.K + 16u * ck : 0xffffffffu;
    }
  }

  const int KT = (g.K + IGEMM_BK - 1) / IGEMM_BK;

  // The loads of K slice kt+1 are in flight while slice kt is multiplied; they are staged
  // into the other LDS buffer afterwards.  (A second register set for a two-slice distance
  // costs 70 registers and with them a workgroup per CU, for no gain: the kernel is bound
  // by LDS traffic, 48 KB per K slice and 128 x 128 tile, not by load latency.)
  struct Staged {
    v4i a[RA], w[RW];
    unsigned amask, wmask;  // bit i: chunk i holds real data (else it is staged as zero)
  };
  [[maybe_unused]] Staged R0;

  // Issue the global loads of the next K slice.  Nothing here consumes a loaded value
  // (that would make the wave wait for it): out-of-image taps and out-of-range rows
  // load from a clamped, always valid address and are zeroed when staged into LDS.
  auto gload = [&](Staged &R) {
    if constexpr (SUB) {
      typedef unsigned v4u __attribute__((ext_vector_type(4)));
      // tap of this lane's chunk: taps per slice * slice + (16 * ck) / Ci; at most 31
      const int t = (u_slice << (6 - g.ci_shift)) + sub_h;
      const int tfy = (t * sub_rkx) >> 16, tfx = t - tfy * g.kx;
      const unsigned toff = (unsigned)((tfy * g.W + tfx) * g.Ci);
#pragma unroll
      for (int i = 0; i < RA; i++) {
        const unsigned oob = (unsigned)__builtin_amdgcn_sbfe((int)pinv[i], t, 1);
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, (poff[i] + toff) | oob, 0, 0);
        R.a[i] = (v4i){(int)v.x, (int)v.y, (int)v.z, (int)v.w};
      }
      // weight bytes past the end of a row (K is not a multiple of 64) belong to the next row: out of range instead
      const unsigned wtail = (u_slice * IGEMM_BK + 16 * ck < g.K) ? 0u : 0xffffffffu;
#pragma unroll
      for (int i = 0; i < RW; i++) {
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, woff[i] | wtail, u_slice * IGEMM_BK, 0);
        R.w[i] = (v4i){(int)v.x, (int)v.y, (int)v.z, (int)v.w};
      }
      R.amask = R.wmask = ~0u;
      if (u_slice + 1 < KT) u_slice++;
      return;
    }
    if constexpr (UNI) {
      typedef unsigned v4u __attribute__((ext_vector_type(4)));
      const int soff_a = (u_fy * g.W + u_fx) * g.Ci + u_ci;  // scalar: tap and channel offset of the slice
      const int soff_w = u_slice * IGEMM_BK;
#pragma unroll
      for (int i = 0; i < RA; i++) {
        // all ones if this tap is outside the image for this pixel
        const unsigned oob = (unsigned)__builtin_amdgcn_sbfe((int)pinv[i], u_tap, 1);
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, poff[i] | oob, soff_a, 0);
        R.a[i] = (v4i){(int)v.x, (int)v.y, (int)v.z, (int)v.w};
      }
#pragma unroll
      for (int i = 0; i < RW; i++) {
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, woff[i], soff_w, 0);
        R.w[i] = (v4i){(int)v.x, (int)v.y, (int)v.z, (int)v.w};
      }
      R.amask = R.wmask = ~0u;
      // advance to the next K slice (scalar).  The prefetch runs one slice past the end; that
      // request repeats the last real slice instead, so no address beyond the caller's buffers is
      // ever formed.
      if (u_slice + 1 < KT) {
        u_slice++;
        u_ci += IGEMM_BK;
        if (u_ci >= g.Ci) {
          u_ci = 0;
          u_tap++;
          if (++u_fx == g.kx) { u_fx = 0; ++u_fy; }
        }
      }
      return;
    }
    unsigned amask = 0, wmask = 0;
#pragma unroll
    for (int i = 0; i < RA; i++) {
      if (GATHER == GATHER_CHUNK16) {
        const int iy = iy0[i] + fy, ix = ix0[i] + fx;
        const bool ok = kpos < g.K && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
        const long long off = ok ? abase[i] + ((long long)iy * g.W + ix) * g.Ci + ci : 0;
        R.a[i] = *(const v4i *)(g.in + off);
        amask |= (unsigned)ok << i;
      } else {
        int bfy = fy, bfx = fx, bci = ci;
        unsigned bytes[4] = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 16; j++) {
          if (kpos + j < g.K) {
            const int iy = iy0[i] + bfy, ix = ix0[i] + bfx;
            if ((unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W)
              bytes[j >> 2] |= (unsigned)g.in[abase[i] + ((long long)iy * g.W + ix) * g.Ci + bci] << (8 * (j & 3));
          }
          if (++bci == g.Ci) {
            bci = 0;
            if (++bfx == g.kx) { bfx = 0; ++bfy; }
          }
        }
        R.a[i] = (v4i){(int)bytes[0], (int)bytes[1], (int)bytes[2], (int)bytes[3]};
        amask |= 1u << i;
      }
    }
#pragma unroll
    for (int i = 0; i < RW; i++) {
      const int n = n0 + wchan[i];
      if (GATHER == GATHER_CHUNK16) {
        const bool ok = wact[i] && n < g.N && kpos < g.K;
        const long long off = ok ? (long long)n * g.K + kpos : 0;
        R.w[i] = *(const v4i *)(g.w + off);
        wmask |= (unsigned)ok << i;
      } else {
        unsigned bytes[4] = {0, 0, 0, 0};
        if (wact[i] && n < g.N) {
          const int8_t *src = g.w + (long long)n * g.K + kpos;
#pragma unroll
          for (int j = 0; j < 16; j++)
            if (kpos + j < g.K) bytes[j >> 2] |= (unsigned)(uint8_t)src[j] << (8 * (j & 3));
        }
        R.w[i] = (v4i){(int)bytes[0], (int)bytes[1], (int)bytes[2], (int)bytes[3]};
        wmask |= 1u << i;
      }
    }
    R.amask = amask;
    R.wmask = wmask;
    // advance to the next K slice
    kpos += IGEMM_BK;
    ci += IGEMM_BK;
    while (ci >= g.Ci) {
      ci -= g.Ci;
      if (++fx == g.kx) { fx = 0; ++fy; }
    }
  };

  // Stage the loaded slice into LDS: activations as a ^ 0x80, invalid chunks as zero
  // (0x80 after the xor); weight bytes also feed the per-row sums.
  // live: the slice is one of the KT real ones (the prefetch runs up to two slices past
  // the end; those are staged but never multiplied, and must not reach the weight sums).
  auto sts = [&](const Staged &R, int buf, bool live) {
#pragma unroll
    for (int i = 0; i < RA; i++) {
      v4i v = R.a[i];
      if (!UNI && !((R.amask >> i) & 1)) v = (v4i){0, 0, 0, 0};
      *(v4i *)&As[buf][lds_off((tid >> 2) + RPP * i, ck)] = v ^ (int)0x80808080;
    }
#pragma unroll
    for (int i = 0; i < RW; i++) {
      v4i v = R.w[i];
      if (!UNI && !((R.wmask >> i) & 1)) v = (v4i){0, 0, 0, 0};
      if (wact[i]) *(v4i *)&Ws[buf][lds_off(wrow[i], ck)] = v;
      if (!UNI || live) {
        wpart[i] = __builtin_amdgcn_sdot4(v.x, 0x01010101, wpart[i], false);
        wpart[i] = __builtin_amdgcn_sdot4(v.y, 0x01010101, wpart[i], false);
        wpart[i] = __builtin_amdgcn_sdot4(v.z, 0x01010101, wpart[i], false);
        wpart[i] = __builtin_amdgcn_sdot4(v.w, 0x01010101, wpart[i], false);
      }
    }
  };

  v4i acc[TN][TM];
#pragma unroll
  for (int t = 0; t < TN; t++)
#pragma unroll
    for (int s = 0; s < TM; s++) acc[t][s] = (v4i){0, 0, 0, 0};

  // fragment rows of this lane
  const int l16 = lane & 15, lgrp = lane >> 4;
  const int wfrag_row0 = wave_n * WN + l16;
  const int afrag_row0 = wave_m * WM + l16;

  auto compute = [&](int cur) {
    v4i wf[TN], af[TM];
#pragma unroll
    for (int t = 0; t < TN; t++) wf[t] = *(const v4i *)&Ws[cur][lds_off(wfrag_row0 + 16 * t, lgrp)];
#pragma unroll
    for (int s = 0; s < TM; s++) af[s] = *(const v4i *)&As[cur][lds_off(afrag_row0 + 16 * s, lgrp)];
#pragma unroll
    for (int t = 0; t < TN; t++)
#pragma unroll
      for (int s = 0; s < TM; s++)
        acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[t], af[s], acc[t][s], 0, 0, 0);
  };
  // Slices past the end are loaded and staged but never multiplied: no branches needed.
  // (The loop is kept rolled: unrolled by two it costs 60 more registers and a workgroup per CU.)
  for (int c = tid; c < BN; c += NTH) {
    const int n = n0 + c;
    int b = 0;
    bn_t kv = 0, lv = 0;
    if (n < g.N) {
      if (g.bias) b = (MODE == EPI_OUT32) ? ((const int *)g.bias)[n] : (int)g.bias[n];
      if (MODE == EPI_BN) {
        kv = e.k[n];
        lv = e.lambda[n];
      }
    }
    cbias[c] = b;
    if (MODE == EPI_BN) {
      ck_[c] = kv;
      cl_[c] = lv;
    }
  }
  if constexpr (ONEPASS > 0) {
    Staged R[ONEPASS];
#pragma unroll
    for (int kt = 0; kt < ONEPASS; kt++)
      if (kt < KT) gload(R[kt]);
#pragma unroll
    for (int kt = 0; kt < ONEPASS; kt++)
      if (kt < KT) sts(R[kt], kt, true);
    __syncthreads();
#pragma unroll
    for (int kt = 0; kt < ONEPASS; kt++)
      if (kt < KT) compute(kt);
  } else {
    gload(R0);
    sts(R0, 0, true);
    __syncthreads();
#pragma unroll 1
    for (int kt = 0; kt < KT; kt++) {
      gload(R0);                            // slice kt + 1
      compute(kt & 1);                      // slice kt
      sts(R0, (kt + 1) & 1, kt + 1 < KT);
      __syncthreads();
    }
  }
  // ---- per-row weight sums -> LDS (indexed by LDS row) ---------------------
#pragma unroll
  for (int i = 0; i < RW; i++) {
    int v = wpart[i];
    v += __shfl_xor(v, 1);
    v += __shfl_xor(v, 2);
    if (wact[i] && ck == 0) wsum[wrow[i]] = v;
  }
  __syncthreads();

  // ---- epilogue ------------------------------------------------------------
  igemm_epilogue<TN, TM, MODE>(acc, g, e, m0, n0, wave_m * WM, wave_n * WN, lane, wsum, cbias, ck_, cl_);
}
