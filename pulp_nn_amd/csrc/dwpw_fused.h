// Depthwise 3x3 + pointwise 1x1 in one kernel: the block of a MobileNet-style network.
//
// The reference runs the two layers as separate calls with the depthwise result written to memory in
// HWC (32bit/src/pulp_nn_depthwise_generic.c:179) and read back pixel by pixel by the next layer
// (pulp_nn_pointwise_HoWo_parallel.c:103).  Here a workgroup computes the depthwise layer for a tile of
// output pixels and all channels into LDS, already in the form the matrix cores take as the pointwise
// layer's activation operand (a ^ 0x80, K = channels contiguous per pixel, 64-byte K slices with the
// chunk swizzle of igemm.h), and multiplies it by the pointwise weights from there: the intermediate
// tensor never exists in memory, and a block is one launch instead of two.  Both layers apply their
// own requantisation exactly as the separate kernels do (the depthwise output is rounded to uint8
// before it enters the pointwise layer), so the result is bit-identical to the two-call sequence.
//
// Stage 1 (depthwise, HWC input, padding 1, stride 1 or 2): the register-resident scheme of
// dw3x3_rows_kernel.  A wave takes 64 channels x R output rows of full width (with fewer than 64
// channels: 64 / C groups of R rows, C channels each); a lane quad loads a dword (its four channels)
// of four neighbouring pixels each and transposes it in registers into four pixels per channel; the
// 3x3 windows are v_dot4 on byte windows; the requantised bytes are transposed back to four channels
// of one pixel per lane and written to LDS.
// Stage 2 (pointwise): blocks of 16*TMB pixels x 64 channels, dealt to the waves; the weight fragments of a
// block are fetched straight from global memory in MFMA operand layout, KP slices of K per pass (the first pass
// of a wave's first block is requested before stage 1, so that it arrives while stage 1 runs; a wave's next
// blocks of the same channel group reuse the fragments when one pass covers all of K); 128 * sum_k w comes from
// one more MFMA per fragment against a matrix of ones; the per-channel constants of both layers are cached in
// LDS; both epilogues pick their requantisation branch at run time.
//
// Several blocks of one shape (stride 1, as many channels out as in) run back to back in one launch: a tile is
// then made of whole images, so that the 3x3 window of a pixel never leaves it; the epilogue of a block writes
// its bytes to LDS in HWC order instead of to memory, the depthwise stage of the next block reads them from
// there, and only the last block's output leaves the chip.  The blocks' parameters are an array in the kernel
// arguments.  The weight fragments of a wave's first stage-2 block of the next block are requested behind the
// MFMAs of its last one in this block: they travel during the epilogue, the barrier and the next depthwise stage.
#pragma once
#include "depthwise.h"
#include "igemm.h"

#define DWPW_MAX_BLOCKS 8  // blocks of one launch (pulp_nn_hip_dw_pw_chain_hwc)
#define DWPW_YPAD 64        // padding bytes per pixel of a block's output kept in LDS for the next block

// one depthwise + pointwise block
struct DwPwBlock {
  const int8_t *dw_wt;    // [C][3][3]
  const int8_t *dw_bias;  // int8 [C] or null
  const int8_t *pw_w;     // [Co][C]
  const int8_t *pw_bias;  // int8 [Co] or null
  EpiArgs e_dw, e_pw;     // k, lambda, multiplier, shift of either layer
  int mode_dw, mode_pw;   // requantisation branch of either layer (EPI_BN, EPI_MULT, EPI_RAW)
};

struct DwPwGeom {
  const uint8_t *in;      // HWC [B][H][W][C]
  uint8_t *out;           // HWC [B][Ho][Wo][Co]
  int B, C, H, Ho, Co;
  int M;                  // B * Ho * Wo output pixels
  int BM;                 // pixels per tile: a multiple of 64 and of the pixels of a stage-1 item
  int KT;                 // 64-byte K slices: ceil(C / 64)
  int nsplit;             // workgroups that share a pixel tile, each computing Co / 64 / nsplit channel blocks
  FastDiv d_howo;         // division by Ho * Wo
  // More than one block (stride 1, C == Co, tiles of whole images, nsplit == 1): block j + 1 reads the output of
  // block j from LDS, where block j's epilogue left it in HWC order; only the last block writes to memory.
  int nblocks;
  DwPwBlock blk[DWPW_MAX_BLOCKS];
};

// LDS bytes of the activation operand: 64-byte K slices; with 16 or 32 channels a pixel's row is just its
// C bytes (the MFMA still multiplies 64 bytes of K, but the weights of the missing ones are zero, so the lanes
// that would fetch them may read any bytes at all: they re-read the real ones)
__host__ __device__ static inline int dwpw_lds_bytes(int BM, int C) { return C < 64 ? BM * C : BM * ((C + 63) / 64) * 64; }
// ... and of the pointwise layer's per-channel constants (bias, k, lambda) behind it, for nch channels
__host__ __device__ static inline int dwpw_const_bytes(int nch) { return nch * (4 + 2 * (int)sizeof(bn_t)); }

// WB, R, S: input width, output rows per stage-1 item, stride.  NWV: waves per workgroup.  TMB: a stage-2 block
// is 16*TMB pixels x 64 channels.  KP: K slices whose weight fragments a wave holds at once (a pass over K).
// The requantisation branches of both layers are run-time switches: one kernel per geometry, not nine.
// CHAIN: g.nblocks blocks back to back; otherwise the one block g.blk[0], with nothing of the chain's loop left.
template <int WB, int R, int S, int NWV, int TMB, int KP, bool CHAIN = false>
__global__ __launch_bounds__(64 * NWV) void dwpw_fused_kernel(DwPwGeom g)
{
  constexpr int DWPW_WAVES = NWV;
  constexpr int BP = 16 * TMB;          // pixels of a stage-2 block
  constexpr int RD = WB / 4;            // dwords per input row (per channel, after the transpose)
  constexpr int WO = (WB - 1) / S + 1;  // output columns
  constexpr int XG = WO / 4;            // groups of 4 output columns
  constexpr int NIN = (R - 1) * S + 3;  // input rows behind R output rows
  constexpr int O0 = 3;
  constexpr int NS = (O0 + 3 * S + 2) / 4 + 1;
  static_assert(WB % 4 == 0 && WO % 4 == 0, "whole dwords in, whole groups of 4 columns out");
  extern __shared__ __attribute__((aligned(16))) unsigned char dwpw_lds[];  // [KT][BM rows][64 bytes], or [BM rows][C bytes] for C < 64

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, lgrp = lane >> 4;
  const int tile = blockIdx.x / g.nsplit, part = blockIdx.x - tile * g.nsplit;
  const int m0 = tile * g.BM;
  const int HoWo = g.Ho * WO;
  const bool narrow = g.C < 64;                 // rows of C bytes instead of 64-byte K slices

  const int MB = g.BM / BP;                     // pixel blocks of the tile
  const int NBT = (g.Co + 63) / 64;             // channel blocks of the layer
  const int nb_per = (NBT + g.nsplit - 1) / g.nsplit;
  const int nb_lo = part * nb_per, nb_hi = min(NBT, nb_lo + nb_per);
  const int nblk = MB * max(nb_hi - nb_lo, 0);  // blocks of this workgroup, dealt to the waves in turn
  const int nch = max(nb_hi - nb_lo, 0) * 64;
  int *c_bias = (int *)(dwpw_lds + dwpw_lds_bytes(g.BM, g.C));
  bn_t *c_k = (bn_t *)(c_bias + nch), *c_l = c_k + nch;
  // the output of a block that another block follows: [tile pixel][Co + DWPW_YPAD] bytes, the next block's HWC input
  unsigned char *ylds = dwpw_lds + dwpw_lds_bytes(g.BM, g.C) + dwpw_const_bytes(nch);
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};

  // weight fragment t of channel block nb: row i of the fragment is channel nb*64 + (i/4)*16 + 4*t + i%4, so that a
  // lane ends up with 16 consecutive channels (the order igemm.h uses)
  auto load_w = [&](const int8_t *pw_w, v4i (&wf)[KP][4], int nb, int kt0) {
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc((void *)pw_w, 0, (unsigned)g.Co * (unsigned)g.C, 0x00020000);
#pragma unroll
    for (int kk = 0; kk < KP; kk++)
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const int n = nb * 64 + (l16 >> 2) * 16 + 4 * t + (l16 & 3);
        const int kb = 64 * (kt0 + kk) + 16 * lgrp;
        const unsigned off = (n < g.Co && kb < g.C && kt0 + kk < g.KT) ? (unsigned)(n * g.C + kb) : 0xffffffffu;
        const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, off, 0, 0);
        wf[kk][t] = (v4i){(int)v.x, (int)v.y, (int)v.z, (int)v.w};
      }
  };
  v4i wf[KP][4];
  int wf_nb = -1;  // channel block whose first-pass fragments wf holds
  const int nblocks = CHAIN ? g.nblocks : 1;
#pragma unroll 1
  for (int j = 0; j < nblocks; j++) {
    const DwPwBlock &P = g.blk[CHAIN ? j : 0];
    const bool first = !CHAIN || j == 0, last = !CHAIN || j == nblocks - 1;

    // ---- stage 2 set-up ------------------------------------------------------------------------------------
    // The pointwise layer's per-channel constants of this workgroup's channel blocks go to LDS (behind the
    // activation operand), where every stage-2 block's epilogue reads them.  Their loads are issued first and the
    // weight fragments' behind them: loads complete in order, so the wait for the constants leaves the fragments
    // in flight.
    constexpr int NCI = (1024 + 64 * DWPW_WAVES - 1) / (64 * DWPW_WAVES);  // at most 1024 output channels
    int cb_[NCI];
    bn_t ck_[NCI], cl_[NCI];
#pragma unroll
    for (int q = 0; q < NCI; q++) {
      const int c = tid + q * 64 * DWPW_WAVES, n = nb_lo * 64 + c;
      const bool ok = c < nch && n < g.Co;
      cb_[q] = (P.pw_bias && ok) ? (int)P.pw_bias[n] : 0;
      ck_[q] = (P.mode_pw == EPI_BN && ok) ? P.e_pw.k[n] : (bn_t)0;
      cl_[q] = (P.mode_pw == EPI_BN && ok) ? P.e_pw.lambda[n] : (bn_t)0;
    }
    // this wave's first stage-2 block: its weight fragments are requested now (first block of the launch; for the
    // others the request went out behind the MFMAs of the block before)
    if (first && wave < nblk) {
      wf_nb = nb_lo + wave / MB;
      load_w(P.pw_w, wf, wf_nb, 0);
    }
#pragma unroll
    for (int q = 0; q < NCI; q++) {
      const int c = tid + q * 64 * DWPW_WAVES;
      if (c < nch) {
        c_bias[c] = cb_[q];
        c_k[c] = ck_[q];
        c_l[c] = cl_[q];
      }
    }

    // ---- stage 1: depthwise into LDS ---------------------------------------------------------------------
    {
      const int CGN = g.C >= 64 ? g.C / 64 : 1;  // channel groups
      const int LG = g.C >= 64 ? 1 : 64 / g.C;   // row groups inside a wave (fewer than 64 channels)
      const int item_px = R * LG * WO;
      const int nitems = (g.BM / item_px) * CGN;
      const unsigned sel1 = quad_sel1(lane), sel2 = quad_sel2(lane);
      for (int it = wave; it < nitems; it += DWPW_WAVES) {
        const int cg = it % CGN, seg = it / CGN;
        const int lg = g.C >= 64 ? 0 : lane / g.C;
        const int ch = g.C >= 64 ? cg * 64 + lane : lane % g.C;
        const int mi = m0 + seg * item_px;  // first pixel of the item (all of it in one image)
        if (mi >= g.M) break;
        const int b = (int)fastdiv((unsigned)mi, g.d_howo);
        const int oy0 = (mi - b * HoWo) / WO + lg * R;  // first output row of this lane's group
        unsigned row[NIN][RD];
        // the image this item lies in: in memory for the first block, else where the block before left it (a tile of
        // several blocks is made of whole images, stride 1: image (b - first image of the tile) of the tile)
        // (in LDS a pixel takes 64 bytes more than its channels: with the power-of-two pitch the four pixels a lane
        // quad reads here, and the pixels a store of the epilogue writes, would all start in the same bank)
        const int pitch = first ? g.C : g.C + DWPW_YPAD;
        const uint8_t *img = first ? g.in + (long long)b * g.H * WB * g.C
                                   : ylds + (long long)(b - (int)fastdiv((unsigned)m0, g.d_howo)) * g.H * WB * pitch;
        const uint8_t *src = img + (lane & 3) * pitch + (ch & ~3);
#pragma unroll
        for (int r = 0; r < NIN; r++) {
          const int iy = oy0 * S - 1 + r;
          const bool ok = (unsigned)iy < (unsigned)g.H;
          const uint8_t *rp = src + (long long)min(max(iy, 0), g.H - 1) * WB * pitch;
#pragma unroll
          for (int d = 0; d < RD; d++) {
            const unsigned v = *(const unsigned *)(rp + (long long)(4 * d) * pitch);
            row[r][d] = ok ? v : 0u;
          }
        }
#pragma unroll
        for (int r = 0; r < NIN; r++)
#pragma unroll
          for (int d = 0; d < RD; d++) row[r][d] = quad_transpose4x4_perm(row[r][d], sel1, sel2) ^ 0x80808080u;
        unsigned wA[3], wB[3];
        int wsum = 0;
#pragma unroll
        for (int i = 0; i < 3; i++) {
          const int8_t *p = P.dw_wt + (long long)ch * 9 + 3 * i;
          const unsigned k0 = (uint8_t)p[0], k1 = (uint8_t)p[1], k2 = (uint8_t)p[2];
          wA[i] = k0 | (k1 << 8) | (k2 << 16);
          wB[i] = wA[i] << 8;
          wsum += (int)p[0] + (int)p[1] + (int)p[2];
        }
        const int corr = 128 * wsum + (P.dw_bias ? (int)P.dw_bias[ch] : 0);
        bn_t kk = 0, ll = 0;
        if (P.mode_dw == EPI_BN) {
          kk = P.e_dw.k[ch];
          ll = P.e_dw.lambda[ch];
        }
        const int dw_mult = P.e_dw.mult, dw_shift = P.e_dw.shift;
        const bool fastq = (P.mode_dw == EPI_BN) ? __all(bn_k_small(kk)) : (dw_shift >= 16);
        // after the quad transpose this lane holds channels (ch & ~3) .. + 3 of pixel column 4*xg + lane%4:
        // one dword of the activation operand, K slice (ch / 64), 16-byte chunk (ch % 64) / 16
        const int c4 = ch & ~3;
        unsigned char *abase = narrow ? dwpw_lds + c4 : dwpw_lds + (c4 >> 6) * (g.BM * 64) + (c4 & 15);
        const int chunk = (c4 & 63) >> 4;
        const int pl0 = seg * item_px + lg * R * WO + (lane & 3);  // tile-local pixel of row 0, column lane % 4
        auto body = [&](auto md, auto fq) {
          constexpr int MODE_DW = decltype(md)::value;
          constexpr bool FASTQ = decltype(fq)::value;
#pragma unroll
          for (int ro = 0; ro < R; ro++) {
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
              unsigned packed = requant4_same<MODE_DW, FASTQ>(acc[0], acc[1], acc[2], acc[3], kk, ll, dw_mult, dw_shift);
              packed = quad_transpose4x4_perm(packed, sel1, sel2) ^ 0x80808080u;
              const int pl = pl0 + ro * WO + 4 * xg;
              *(unsigned *)(abase + (narrow ? pl * g.C : pl * 64 + ((chunk ^ ((pl >> 1) & 3)) << 4))) = packed;
            }
          }
        };
        if (P.mode_dw == EPI_BN) {
          if (fastq) body(std::integral_constant<int, EPI_BN>{}, std::true_type{});
          else body(std::integral_constant<int, EPI_BN>{}, std::false_type{});
        } else if (P.mode_dw == EPI_MULT) {
          if (fastq) body(std::integral_constant<int, EPI_MULT>{}, std::true_type{});
          else body(std::integral_constant<int, EPI_MULT>{}, std::false_type{});
        } else {
          body(std::integral_constant<int, EPI_RAW>{}, std::false_type{});
        }
      }
    }
    __syncthreads();

    // ---- stage 2: pointwise from LDS ---------------------------------------------------------------------
    const int swz = (lgrp ^ ((l16 >> 1) & 3)) << 4;
    // narrow rows: chunk lgrp of a row if it exists, else chunk 0 (multiplied by zero weights)
    const int nar_off = l16 * g.C + ((16 * lgrp < g.C) ? 16 * lgrp : 0);
    const int pw_mult = P.e_pw.mult, pw_shift = P.e_pw.shift;
    for (int blk = wave; blk < nblk; blk += DWPW_WAVES) {
      const int mb = blk % MB, nb = nb_lo + blk / MB;
      v4i acc[4][TMB], wacc[4];
#pragma unroll
      for (int t = 0; t < 4; t++) {
        wacc[t] = (v4i){0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < TMB; s++) acc[t][s] = (v4i){0, 0, 0, 0};
      }
      for (int kt0 = 0; kt0 < g.KT; kt0 += KP) {
        // (the first pass of the first block was requested before stage 1; a wave's next blocks of the same channel
        // block re-use the fragments when one pass covers K)
        if (kt0 > 0 || wf_nb != nb || g.KT > KP) {
          load_w(P.pw_w, wf, nb, kt0);
          wf_nb = kt0 == 0 ? nb : -1;
        }
#pragma unroll
        for (int kk = 0; kk < KP; kk++) {
          if (kt0 + kk < g.KT) {
            const unsigned char *ab = narrow ? dwpw_lds + mb * BP * g.C + nar_off
                                             : dwpw_lds + (kt0 + kk) * (g.BM * 64) + (mb * BP + l16) * 64 + swz;
            const int sstep = narrow ? 16 * g.C : 1024;  // 16 rows on
            v4i af[TMB];
#pragma unroll
            for (int s = 0; s < TMB; s++) af[s] = *(const v4i *)(ab + s * sstep);
#pragma unroll
            for (int t = 0; t < 4; t++) {
#pragma unroll
              for (int s = 0; s < TMB; s++) acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[kk][t], af[s], acc[t][s], 0, 0, 0);
              wacc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[kk][t], ones, wacc[t], 0, 0, 0);
            }
          }
        }
      }
      // the last stage-2 block of this wave in this block of the chain: the weight fragments of its first one in the
      // next block are requested now, so that they travel while the epilogue, the barrier and the next depthwise
      // stage run
      if (!last && blk + DWPW_WAVES >= nblk) {
        wf_nb = nb_lo + wave / MB;
        load_w(g.blk[CHAIN ? j + 1 : 0].pw_w, wf, wf_nb, 0);
      }
      // epilogue: acc[t][s][r] = channel cb + 4*t + r of pixel m0 + mb*BP + 16*s + l16; wacc[t][r] = sum of that channel's weights
      const int cb = nb * 64 + lgrp * 16;
      const bool acc24 = g.C <= 256;  // |acc| <= K * 255 * 128 + 128 < 2^23
      unsigned packed[TMB][4];
      auto requantise = [&](auto md) {
        constexpr int MODE_PW = decltype(md)::value;
#pragma unroll
        for (int t = 0; t < 4; t++) {
          int corr[4];
          bn_t kk[4], ll[4];
          bool ks = true;
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const int c = cb + 4 * t + r - nb_lo * 64;  // channel inside this workgroup's range (constants past Co are zero)
            kk[r] = (MODE_PW == EPI_BN) ? c_k[c] : (bn_t)0;
            ll[r] = (MODE_PW == EPI_BN) ? c_l[c] : (bn_t)0;
            ks = ks && bn_k_small(kk[r]);
            corr[r] = c_bias[c] + 128 * wacc[t][r];
          }
          const bool k_small = __all(ks);
#pragma unroll
          for (int s = 0; s < TMB; s++) {
            const int a0 = acc[t][s][0] + corr[0], a1 = acc[t][s][1] + corr[1];
            const int a2 = acc[t][s][2] + corr[2], a3 = acc[t][s][3] + corr[3];
            packed[s][t] = acc24 ? requant4<MODE_PW, true>(a0, a1, a2, a3, kk, ll, k_small, pw_mult, pw_shift)
                                 : requant4<MODE_PW, false>(a0, a1, a2, a3, kk, ll, k_small, pw_mult, pw_shift);
          }
        }
      };
      if (P.mode_pw == EPI_BN) requantise(std::integral_constant<int, EPI_BN>{});
      else if (P.mode_pw == EPI_MULT) requantise(std::integral_constant<int, EPI_MULT>{});
      else requantise(std::integral_constant<int, EPI_RAW>{});
#pragma unroll
      for (int s = 0; s < TMB; s++) {
        const int pl = mb * BP + 16 * s + l16;  // tile-local pixel
        if (m0 + pl < g.M && cb < g.Co) {
          const v4i v = {(int)packed[s][0], (int)packed[s][1], (int)packed[s][2], (int)packed[s][3]};
          if (last) *(v4i *)(g.out + (long long)(m0 + pl) * g.Co + cb) = v;
          else *(v4i *)(ylds + pl * (g.Co + DWPW_YPAD) + cb) = v;
        }
      }
    }
    // the next block reads this one's output and rewrites the activation operand and the constants
    if (!last) __syncthreads();
  }
}
