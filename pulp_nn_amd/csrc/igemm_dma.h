// Implicit-GEMM kernel for large standard convolutions (and any GEMM of the same shape) whose
// input channels are a multiple of 128: the MFMA-bound case of
// 32bit/src/pulp_nn_conv_Ho_parallel.c:76-183 + pulp_nn_matmul.c:53-216.
//
// Same arithmetic as igemm_kernel (activations as a ^ 0x80, 128 * sum_k w added back, identical
// epilogue); what differs is how the operands reach the matrix cores:
//   * tile of 256 pixels x 256 channels, eight waves of 128 x 64 (32 MFMAs per 12 fragment reads),
//     two waves per SIMD with up to 256 registers each;
//   * K slices of 128 bytes (a pixel's slice is one whole 128-byte line of the HWC input), double
//     buffered in LDS: one barrier per 64 MFMAs of a wave;
//   * the slices travel HBM/L2 -> LDS with buffer loads that write LDS directly
//     (buffer_load_dwordx4 ... lds): no staging registers, no LDS store instructions, and the
//     loads of slice kt+1 are in flight for the whole of slice kt.  A wave's load writes 1 KB of
//     consecutive LDS (lane l at 16*l), so the XOR swizzle that makes the fragment reads
//     conflict-free is applied to the global address each lane fetches instead of to the LDS
//     address it writes;
//   * the ^ 0x80 is applied to the activation fragments after they are read from LDS (an
//     out-of-image tap is an out-of-range buffer load, which writes zeros: 0x80 after the xor);
//   * the weight sums come from the matrix core as well: a weight fragment times a matrix of ones
//     gives the sums of its 16 rows.  Each wave does that for two of its four fragments; the two
//     waves that share the fragments (same channels, other pixel half) split them between them.
//     (v_dot4 on the fragments costs several times the issue slots and holds up the MFMAs behind it:
//     16 % of the main loop.)
#pragma once
#include "igemm.h"

#define IGD_THREADS 512
#define IGD_SUB (256 * 64)  // bytes of one sub-slice (64 bytes of K) of 256 rows

// dynamic LDS: activations [2 buffers][2 sub-slices][16 KB], weights the same, then the per-channel
// constants of the tile
static inline int igd_lds_bytes() { return 8 * IGD_SUB + 256 * (4 + 4 + 2 * (int)sizeof(bn_t)); }

template <int MODE>
__global__ __launch_bounds__(IGD_THREADS, 1) void igemm_dma_kernel(ConvGeom g, EpiArgs e)
{
  constexpr int TM = 8, TN = 4, WM = 128, WN = 64, BM = 256, BN = 256;
  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char igd_lds[];
  unsigned char *As = igd_lds;
  unsigned char *Ws = igd_lds + 4 * IGD_SUB;
  int *wsum = (int *)(igd_lds + 8 * IGD_SUB);
  int *cbias = wsum + BN;
  bn_t *ck_ = (bn_t *)(cbias + BN);
  bn_t *cl_ = ck_ + BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave & 1, wave_n = wave >> 1;
  const int l16 = lane & 15, lgrp = lane >> 4;

  const int tile = xcd_remap(blockIdx.x, g.tiles_total);
  const int tile_m = (int)fastdiv((unsigned)tile, g.d_tiles_n);
  const int m0 = tile_m * BM;
  const int n0 = (tile - tile_m * g.tiles_n) * BN;

  // ---- what this lane fetches ------------------------------------------------------------------
  // A load instruction of wave w fills LDS rows 16*rb .. 16*rb+15 of one sub-slice, rb = 2*w + j:
  // lane l writes slot l%4 of row 16*rb + l/4, which has to hold K chunk (l%4) ^ ((row/2)%4).
  const unsigned OOB = 0x80000000u;  // offsets stay below 2^31 (checked by the host), so this bit puts a load out of range
  const unsigned shift = (unsigned)((g.pt * g.W + g.pl) * g.Ci);
  const unsigned batch = (unsigned)g.batch;
  const __amdgpu_buffer_rsrc_t rsrc_a =
      __builtin_amdgcn_make_buffer_rsrc((void *)(g.in - shift), 0, shift + batch * (unsigned)g.in_img, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)g.w, 0, (unsigned)g.N * (unsigned)g.K, 0x00020000);
  unsigned poff[2], pinv[2], woff[2];
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int row = 16 * (2 * wave + j) + (lane >> 2);
    const unsigned chunk = (unsigned)((lane & 3) ^ ((row >> 1) & 3));
    const int m = m0 + row;
    poff[j] = OOB;
    pinv[j] = 0;
    if (m < g.M) {
      const int b = (int)fastdiv((unsigned)m, g.d_howo), rem = m - b * g.HoWo;
      const int oy = (int)fastdiv((unsigned)rem, g.d_wo), ox = rem - oy * g.Wo;
      poff[j] = (unsigned)b * (unsigned)g.in_img + (unsigned)((oy * g.sy * g.W + ox * g.sx) * g.Ci) + 16u * chunk;
      for (int fy_ = 0, t = 0; fy_ < g.ky; fy_++)
        for (int fx_ = 0; fx_ < g.kx; fx_++, t++) {
          const int iy = oy * g.sy - g.pt + fy_, ix = ox * g.sx - g.pl + fx_;
          if ((unsigned)iy >= (unsigned)g.H || (unsigned)ix >= (unsigned)g.W) pinv[j] |= 1u << t;
        }
    }
    // weight rows sit in LDS in fragment order (see igemm_kernel): LDS row p holds channel
    // (p/64)*64 + ((p%16)/4)*16 + 4*((p%64)/16) + p%4
    const int pp = row % WN, t = pp >> 4, r16 = pp & 15;
    const int n = n0 + (row / WN) * WN + (r16 >> 2) * (4 * TN) + 4 * t + (r16 & 3);
    woff[j] = n < g.N ? (unsigned)n * (unsigned)g.K + 16u * chunk : OOB;
  }

  // scalar walk over the K slices: (tap, first channel) of the next slice to request
  int u_tap = 0, u_fx = 0, u_fy = 0, u_ci = 0, u_slice = 0;
  const int KT = g.K / 128;
  auto dma = [&](int buf) {
    const int soff_a = (u_fy * g.W + u_fx) * g.Ci + u_ci;
    const int soff_w = u_slice * 128;
    // (the second half of a line is reached through the scalar offset: an instruction's immediate offset
    // would also move the LDS address it writes)
    unsigned char *a_dst = As + buf * 2 * IGD_SUB + wave * 2048;
    unsigned char *w_dst = Ws + buf * 2 * IGD_SUB + wave * 2048;
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const unsigned oob = (unsigned)__builtin_amdgcn_sbfe((int)pinv[j], u_tap, 1) & OOB;
      const int va = (int)(poff[j] | oob);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)(a_dst + 1024 * j), 16, va, soff_a, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)(a_dst + 1024 * j + IGD_SUB), 16, va, soff_a + 64, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr_t)(w_dst + 1024 * j), 16, (int)woff[j], soff_w, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr_t)(w_dst + 1024 * j + IGD_SUB), 16, (int)woff[j], soff_w + 64, 0, 0);
    }
    u_slice++;
    u_ci += 128;
    if (u_ci >= g.Ci) {
      u_ci = 0;
      u_tap++;
      if (++u_fx == g.kx) { u_fx = 0; ++u_fy; }
    }
  };

  dma(0);

  // per-channel constants of the tile, fetched while the first slice is on its way
  for (int c = tid; c < BN; c += IGD_THREADS) {
    const int n = n0 + c;
    int b = 0;
    bn_t kv = 0, lv = 0;
    if (n < g.N) {
      if (g.bias) b = (int)g.bias[n];
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

  v4i acc[TN][TM];
#pragma unroll
  for (int t = 0; t < TN; t++)
#pragma unroll
    for (int s = 0; s < TM; s++) acc[t][s] = (v4i){0, 0, 0, 0};
  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
  v4i wacc[2] = {(v4i){0, 0, 0, 0}, (v4i){0, 0, 0, 0}};

  // fragment addresses of this lane: row r of a sub-slice at 64*r, chunk c of it in slot c ^ ((r/2)%4)
  const int swz = (lgrp ^ ((l16 >> 1) & 3)) << 4;
  const int a_lane = (wave_m * WM + l16) * 64 + swz;
  const int w_lane = (wave_n * WN + l16) * 64 + swz;

#pragma unroll 1
  for (int kt = 0; kt < KT; kt++) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this lane's part of slice kt has landed
    __syncthreads();                     // ... everybody's has, and everybody is done reading the other buffer
    if (kt + 1 < KT) dma((kt + 1) & 1);
    const unsigned char *Ab = As + (kt & 1) * 2 * IGD_SUB + a_lane;
    const unsigned char *Wb = Ws + (kt & 1) * 2 * IGD_SUB + w_lane;
    // both sub-slices' activation fragments are requested before the first MFMA, so that the second
    // sub-slice's arrive while the first is multiplied
    v4i wf[TN], af0[TM], af1[TM];
#pragma unroll
    for (int t = 0; t < TN; t++) wf[t] = *(const v4i *)(Wb + t * 1024);
#pragma unroll
    for (int s = 0; s < TM; s++) af0[s] = *(const v4i *)(Ab + s * 1024);
#pragma unroll
    for (int s = 0; s < TM; s++) af1[s] = *(const v4i *)(Ab + IGD_SUB + s * 1024);
    auto multiply = [&](v4i (&af)[TM]) {
#pragma unroll
      for (int s = 0; s < TM; s++) {
        const v4i a = af[s] ^ (int)0x80808080;
#pragma unroll
        for (int t = 0; t < TN; t++) acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[t], a, acc[t][s], 0, 0, 0);
      }
      // (a select, not a branch: wave_m is uniform, and a branch here splits the loop body)
      const v4i ws0 = wave_m ? wf[2] : wf[0], ws1 = wave_m ? wf[3] : wf[1];
      wacc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ws0, ones, wacc[0], 0, 0, 0);
      wacc[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ws1, ones, wacc[1], 0, 0, 0);
    };
    multiply(af0);
#pragma unroll
    for (int t = 0; t < TN; t++) wf[t] = *(const v4i *)(Wb + IGD_SUB + t * 1024);
    multiply(af1);
  }

  // ---- per-row weight sums -> LDS (indexed by LDS row) -------------------------------------------
  // wacc[i][r] of a lane = sum of LDS weight row 16*t + 4*(lane/16) + r of this wave's channels, t = 2*wave_m + i
  if (l16 == 0) {
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int r = 0; r < 4; r++) wsum[wave_n * WN + 16 * (2 * wave_m + i) + 4 * lgrp + r] = wacc[i][r];
  }
  __syncthreads();

  igemm_epilogue<TN, TM, MODE>(acc, g, e, m0, n0, wave_m * WM, wave_n * WN, lane, wsum, cbias, ck_, cl_);
}
