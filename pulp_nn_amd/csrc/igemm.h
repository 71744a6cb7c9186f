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
#pragma once
#include <type_traits>

#include "memops.h"
#include "requant.h"

enum { GATHER_CHUNK16 = 0, GATHER_BYTES = 1 };
enum { EPI_OUT32 = 3 };  // linear_out_32: int32 accumulators + int32 bias, no requantisation

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
};

#define IGEMM_BK 64
#ifndef IGEMM_MINB
#define IGEMM_MINB 2  // workgroups per CU the register budget is sized for
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

template <int TN, int WAVES_M, int WAVES_N, int GATHER, int MODE, int TM = 4>
__global__ __launch_bounds__(256, IGEMM_MINB) void igemm_kernel(ConvGeom g, EpiArgs e)
{
  constexpr int WM = 16 * TM, WN = 16 * TN;
  constexpr int BM = WM * WAVES_M, BN = WN * WAVES_N;
  constexpr int RA = BM / 64;                    // activation chunks per thread per K slice
  constexpr int RW = (BN * 4 + 255) / 256;       // weight chunks per thread per K slice
  static_assert(WAVES_M * WAVES_N == 4, "256 threads");

  __shared__ __attribute__((aligned(16))) uint8_t As[2][BM * IGEMM_BK];
  __shared__ __attribute__((aligned(16))) int8_t Ws[2][BN * IGEMM_BK];
  __shared__ int wsum[BN];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wave_m = wave % WAVES_M, wave_n = wave / WAVES_M;

  const int tile = xcd_remap(blockIdx.x, g.tiles_total);
  const int m0 = (tile / g.tiles_n) * BM;
  const int n0 = (tile % g.tiles_n) * BN;

  // ---- per-thread gather state -------------------------------------------
  const int ck = tid & 3;  // which 16-byte chunk of the 64-byte K slice
  int iy0[RA], ix0[RA];
  long long abase[RA];
#pragma unroll
  for (int i = 0; i < RA; i++) {
    const int m = m0 + (tid >> 2) + 64 * i;
    if (m < g.M) {
      const int b = m / g.HoWo, rem = m - b * g.HoWo;
      const int oy = rem / g.Wo, ox = rem - oy * g.Wo;
      iy0[i] = oy * g.sy - g.pt;
      ix0[i] = ox * g.sx - g.pl;
      abase[i] = (long long)b * g.in_img;
    } else {
      iy0[i] = -(1 << 28);
      ix0[i] = 0;
      abase[i] = 0;
    }
  }
  // (fy, fx, ci) of byte k = 16*ck of the current K slice
  int kpos = 16 * ck;
  int ci = kpos % g.Ci, tap = kpos / g.Ci;
  int fy = tap / g.kx, fx = tap - fy * g.kx;

  // Weight rows sit in LDS in fragment order: LDS row p = wn*WN + 16*t + i holds
  // channel wn*WN + (i/4)*4*TN + 4*t + (i%4), so that MFMA tile t of a wave reads
  // 16 consecutive LDS rows and each lane ends up with 4*TN consecutive channels.
  int wrow[RW];   // LDS row
  int wchan[RW];  // channel offset inside the tile that this row holds
  bool wact[RW];
  int wpart[RW];
#pragma unroll
  for (int i = 0; i < RW; i++) {
    const int q = tid + 256 * i;
    const int p = q >> 2;
    wrow[i] = p;
    const int pp = p % WN, t = pp >> 4, r16 = pp & 15;
    wchan[i] = (p / WN) * WN + (r16 >> 2) * (4 * TN) + 4 * t + (r16 & 3);
    wact[i] = q < BN * 4;
    wpart[i] = 0;
  }

  // Two register sets: the loads of K slice kt+2 are in flight while slice kt is
  // multiplied and slice kt+1 is staged, so a load has two slices of MFMA work to arrive.
  struct Staged {
    v4i a[RA], w[RW];
    unsigned amask, wmask;  // bit i: chunk i holds real data (else it is staged as zero)
  };
  Staged R0, R1;

  // Issue the global loads of the next K slice.  Nothing here consumes a loaded value
  // (that would make the wave wait for it): out-of-image taps and out-of-range rows
  // load from a clamped, always valid address and are zeroed when staged into LDS.
  auto gload = [&](Staged &R) {
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
  auto sts = [&](const Staged &R, int buf) {
#pragma unroll
    for (int i = 0; i < RA; i++) {
      v4i v = R.a[i];
      if (!((R.amask >> i) & 1)) v = (v4i){0, 0, 0, 0};
      *(v4i *)&As[buf][lds_off((tid >> 2) + 64 * i, ck)] = v ^ (int)0x80808080;
    }
#pragma unroll
    for (int i = 0; i < RW; i++) {
      v4i v = R.w[i];
      if (!((R.wmask >> i) & 1)) v = (v4i){0, 0, 0, 0};
      if (wact[i]) *(v4i *)&Ws[buf][lds_off(wrow[i], ck)] = v;
      wpart[i] = __builtin_amdgcn_sdot4(v.x, 0x01010101, wpart[i], false);
      wpart[i] = __builtin_amdgcn_sdot4(v.y, 0x01010101, wpart[i], false);
      wpart[i] = __builtin_amdgcn_sdot4(v.z, 0x01010101, wpart[i], false);
      wpart[i] = __builtin_amdgcn_sdot4(v.w, 0x01010101, wpart[i], false);
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

  const int KT = (g.K + IGEMM_BK - 1) / IGEMM_BK;
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
  // Slices past the end load nothing (all-zero masks) and stage zeros: no branches needed.
  gload(R0);
  sts(R0, 0);
  gload(R1);
  __syncthreads();
  for (int kt = 0; kt < KT; kt += 2) {
    gload(R0);        // slice kt + 2
    compute(0);       // slice kt
    sts(R1, 1);       // slice kt + 1
    __syncthreads();
    if (kt + 1 >= KT) break;
    gload(R1);        // slice kt + 3
    compute(1);       // slice kt + 1
    sts(R0, 0);       // slice kt + 2
    __syncthreads();
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
  // acc[t][s][r] = channel cb + 4*t + r of pixel m0 + wave_m*WM + 16*s + l16.
  // Channel constants are fetched four channels (one MFMA tile row group) at a time to
  // keep the register footprint of the epilogue below that of the main loop.
  const int cb = wave_n * WN + lgrp * (4 * TN);
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
      const int n = n0 + cb + 4 * t + r;
      int b = 0;
      kk[r] = 0;
      ll[r] = 0;
      if (n < g.N) {
        if (g.bias) b = (MODE == EPI_OUT32) ? ((const int *)g.bias)[n] : (int)g.bias[n];
        if (MODE == EPI_BN) {
          kk[r] = e.k[n];
          ll[r] = e.lambda[n];
        }
      }
      ks = ks && bn_k_small(kk[r]);
      corr[r] = b + 128 * wsum[wave_n * WN + 16 * t + 4 * lgrp + r];
    }
    const bool k_small = __all(ks);  // wave-uniform precondition of the fast batch-norm form
#pragma unroll
    for (int s = 0; s < TM; s++) {
      const int a0 = acc[t][s][0] + corr[0], a1 = acc[t][s][1] + corr[1];
      const int a2 = acc[t][s][2] + corr[2], a3 = acc[t][s][3] + corr[3];
      if constexpr (MODE == EPI_OUT32) {
        const int m = m0 + wave_m * WM + 16 * s + l16;
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
        const int m = m0 + wave_m * WM + 16 * s + l16;
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
