// Weights-stationary streaming kernel for pointwise convolutions whose weight
// matrix is small (K <= 256, N <= 256): the HBM-bound case
// (pulp_nn_pointwise_HoWo_parallel at 28x28x128 -> 256 moves 384 bytes per pixel
// for 65 kop, far below the machine balance of ~625 op/B).
//
// The whole weight matrix sits in LDS in MFMA fragment order for the lifetime of
// a (persistent) workgroup, one per CU, together with the per-channel constants.
// Every wave owns a contiguous run of pixels and streams it 16*TM pixels per step:
// the activation bytes go from HBM straight into registers in the MFMA
// column-operand layout (lane = pixel l%16, 16-byte K chunk l/16), each byte is
// loaded by exactly one wave, and the loads run two steps ahead of the arithmetic.
// A quarter of the waves stages the weights and constants; the others request the
// pixels of their first two steps at once, so that HBM is busy while the workgroup
// sets up.  A step multiplies its pixels against every channel group, requantises,
// gathers the channel groups of a pixel in a per-wave LDS tile and writes whole
// pixel rows, 1 KB contiguous per store instruction.  Two barriers end the set-up;
// there is none in the streaming loop and no im2col.
//
// Everything the compiler has to count is fixed at compile time (loads and stores
// per step, channel groups): loads and stores share one in-order counter on this
// hardware, and only with a known number of stores behind a load can the wait for
// that load leave the stores in flight.
//
// Arithmetic is that of igemm.h: activations as a ^ 0x80 with 128 * sum_k w
// added back (by starting the accumulators at bias + 128 * sum_k w).
#pragma once
#include <type_traits>

#include "igemm.h"
#include "requant.h"

struct PwGeom {
  const uint8_t *in;   // [M][K] pixels, K = Ci contiguous
  const int8_t *w;     // [N][K]
  const int8_t *bias;  // int8 [N] or null
  void *out;           // [M][N]
  int M, N, K;
  int nt;              // write the output with non-temporal stores
  int units;           // ceil(M / 16): 16-pixel units, dealt to the waves in equal contiguous runs
};

// LDS bytes: weights, then k and lambda (bn_t), then corr (int) per channel; with more
// than one channel group per pixel, a private output tile per wave of 16*tm rows of
// N + 16 bytes.
__host__ __device__ static inline int pw_lds_fixed(int tn, int ks, int np, bool bn)
{
  return np * 16 * tn * (ks * 64 + 4 + (bn ? 2 * (int)sizeof(bn_t) : 0));
}
static inline int pw_lds_bytes(int tn, int ks, int np, bool bn, int nw, int tm)
{
  const int n = np * 16 * tn;
  return pw_lds_fixed(tn, ks, np, bn) + (np > 1 ? nw * 16 * tm * (n + 16) : 0);
}

// N == NP * 16 * TN: every lane owns 4*TN real channels of each of the NP channel groups.
template <int TN, int KS, int NP, int MODE, bool WIDE, int TM, int NW>
__global__ __launch_bounds__(64 * NW, NW >= 8 ? 1 : 2) void pw_stream_kernel(PwGeom g, EpiArgs e)
{
  constexpr int PX = 16 * TM;      // pixels per step
  constexpr int CG = 16 * TN;      // channels per group
  constexpr int N = NP * CG;       // output channels
  constexpr bool XP = NP > 1;      // gather the groups of a pixel in LDS before storing
  constexpr int OROW = N + 16;     // row pitch of the output tile: the 16 bytes of padding spread
                                   // the pieces that 16 pixel lanes write at equal channel
                                   // offsets over all banks
  extern __shared__ __attribute__((aligned(16))) unsigned char pw_lds[];
  int8_t *Wl = (int8_t *)pw_lds;
  bn_t *kl = (bn_t *)(pw_lds + N * KS * 64);
  bn_t *ll_ = kl + ((MODE == EPI_BN) ? N : 0);
  int *corr_l = (int *)(ll_ + ((MODE == EPI_BN) ? N : 0));

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
  const int l16 = lane & 15, lgrp = lane >> 4;
  unsigned char *ob = pw_lds + pw_lds_fixed(TN, KS, NP, MODE == EPI_BN) + wave * (PX * OROW);

  // ---- this wave's share of the pixels ---------------------------------------------------
  // A quarter of the waves stages the weights; the others request their first pixels at
  // once, have them by the time the weights are in place and so start streaming about one
  // step earlier.  The 16-pixel units of the launch are dealt evenly to the
  // workgroups and, inside a workgroup, one step's worth (TM units) fewer to each staging
  // wave than the average and the rest evenly to the others, all in contiguous runs, so
  // that all waves finish together.
  constexpr int NWS = NW >= 4 ? NW / 4 : 1;  // staging waves
  const bool stager = wave < NWS;
  const int ub0 = (int)((long long)g.units * blockIdx.x / gridDim.x);
  const int nb = (int)((long long)g.units * (blockIdx.x + 1) / gridDim.x) - ub0;  // units of this workgroup
  // (no handicap when a wave has fewer than three steps anyway: the set-up then dominates)
  const int us = nb / NW >= 3 * TM ? nb / NW - TM : nb / NW;                      // units of a staging wave
  const int rest = nb - NWS * us;                                                 // units of the other waves
  const int u_beg = stager ? wave * us : NWS * us + (int)((long long)rest * (wave - NWS) / (NW - NWS));
  const int u_end = stager ? (wave + 1) * us : NWS * us + (int)((long long)rest * (wave - NWS + 1) / (NW - NWS));
  const int px_end = min((ub0 + u_end) * 16, g.M);
  int px = (ub0 + u_beg) * 16;
  // Unconditional loads from clamped addresses (no per-lane branches, so that all
  // loads of a step are issued back to back and nothing waits on them here):
  // pixels past the end of the run re-read its last pixel and K chunks past the end
  // re-read chunk 0 (their weights are zero).
  auto load_a = [&](v4i (&a)[TM][KS], int p0) {
#pragma unroll
    for (int s = 0; s < TM; s++) {
      const int m = max(min(p0 + 16 * s + l16, px_end - 1), 0);
      const uint8_t *row = g.in + (long long)m * g.K;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const int k = ks * 64 + lgrp * 16;
        a[s][ks] = *(const v4i *)(row + (k < g.K ? k : 0));
      }
    }
  };
  v4i b0[TM][KS], b1[TM][KS], b2[TM][KS];

  if (!stager) {
    load_a(b0, px);
    load_a(b1, px + PX);
  }
  // ---- weights and per-channel constants -> LDS (staging waves) -------------------------
  bool small = true;
  if (stager) {
    // All global loads of the set-up are issued before the first of them is consumed.
    constexpr int SB = 64 * NWS;                   // staging threads
    constexpr int CHUNKS = N * KS * 4;             // 16-byte chunks of the padded weight matrix
    constexpr int CH = (CHUNKS + SB - 1) / SB;     // per thread
    constexpr int NC = (N + SB - 1) / SB;          // channels per thread
    v4i wv[CH];
#pragma unroll
    for (int u = 0; u < CH; u++) {
      // LDS row R = ((p*KS + ks)*TN + t)*16 + i holds channel p*CG + (i/4)*4*TN + 4*t + i%4
      const int q = tid + SB * u, R = q >> 2, c = q & 3;
      const int i = R & 15, t = (R >> 4) % TN, ks = (R / CG) % KS, p = R / (CG * KS);
      const int n = p * CG + (i >> 2) * (4 * TN) + 4 * t + (i & 3);
      const int k = ks * 64 + 16 * c;
      const bool ok = q < CHUNKS && k < g.K;
      wv[u] = *(const v4i *)(g.w + (ok ? (long long)n * g.K + k : 0));
    }
    int bv[NC];
    bn_t kv[NC], lv[NC];
#pragma unroll
    for (int u = 0; u < NC; u++) {
      const int n = min(tid + SB * u, N - 1);
      bv[u] = g.bias ? (int)g.bias[n] : 0;
      if constexpr (MODE == EPI_BN) {
        kv[u] = e.k[n];
        lv[u] = e.lambda[n];
      }
    }
#pragma unroll
    for (int u = 0; u < CH; u++) {
      const int q = tid + SB * u, R = q >> 2, c = q & 3;
      const int k = ((R / CG) % KS) * 64 + 16 * c;
      if (q < CHUNKS) *(v4i *)&Wl[lds_off(R, c)] = (k < g.K) ? wv[u] : (v4i){0, 0, 0, 0};
    }
    // The staging waves request their first two steps only now: the CU's memory pipeline
    // serves requests in order, and their (few, mostly L2-resident) set-up loads were not
    // to queue behind their own pixels from HBM.
    load_a(b0, px);
    load_a(b1, px + PX);
#pragma unroll
    for (int u = 0; u < NC; u++) {
      const int n = tid + SB * u;
      if (n < N) {
        corr_l[n] = bv[u];
        if constexpr (MODE == EPI_BN) {
          kl[n] = kv[u];
          ll_[n] = lv[u];
          small = small && bn_k_small(kv[u]);
        }
      }
    }
  }
  const bool k_small = __syncthreads_and(small);
  // corr = bias + 128 * sum_k w: the row sums of a weight tile are its product with a
  // matrix of ones; each tile has one owner wave and each channel one owner lane.
  for (int tile = wave; tile < NP * TN; tile += NW) {
    const int p = tile / TN, t = tile % TN;
    v4i acc = {0, 0, 0, 0};
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const v4i wf = *(const v4i *)&Wl[lds_off(((p * KS + ks) * TN + t) * 16 + l16, lgrp)];
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, ones, acc, 0, 0, 0);
    }
    if (l16 == 0) {
      v4i *c4 = (v4i *)&corr_l[p * CG + lgrp * (4 * TN) + 4 * t];
      *c4 = *c4 + acc * 128;
    }
  }
  __syncthreads();

  // ---- stream pixels ------------------------------------------------------------------
  // One step: 16 * TM pixels against every channel group.
  auto process = [&](v4i (&a)[TM][KS], int p0, auto nt) {
    constexpr bool NT = decltype(nt)::value;
#pragma unroll
    for (int s = 0; s < TM; s++)
#pragma unroll
      for (int ks = 0; ks < KS; ks++) a[s][ks] ^= (int)0x80808080;

#pragma unroll 1
    for (int p = 0; p < NP; p++) {
      const int cb = p * CG + lgrp * (4 * TN);  // first of this lane's 4*TN channels
      v4i acc[TN][TM];
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int t = 0; t < TN; t++) {
          const v4i wf = *(const v4i *)&Wl[lds_off(((p * KS + ks) * TN + t) * 16 + l16, lgrp)];
          if (ks == 0) {
            // the accumulators start at bias + 128 * sum_k w, fed in as the MFMA addend
            const v4i c4 = *(const v4i *)&corr_l[cb + 4 * t];
#pragma unroll
            for (int s = 0; s < TM; s++) acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, a[s][ks], c4, 0, 0, 0);
          } else {
#pragma unroll
            for (int s = 0; s < TM; s++)
              acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, a[s][ks], acc[t][s], 0, 0, 0);
          }
        }

      bn_t kk[4 * TN], lam[4 * TN];
      if constexpr (MODE == EPI_BN) {
#pragma unroll
        for (int c = 0; c < 4 * TN; c++) {
          kk[c] = kl[cb + c];
          lam[c] = ll_[cb + c];
        }
      }
#pragma unroll
      for (int s = 0; s < TM; s++) {
        unsigned packed[TN];
#pragma unroll
        for (int t = 0; t < TN; t++)
          packed[t] = requant4<MODE, true, WIDE>(acc[t][s][0], acc[t][s][1], acc[t][s][2], acc[t][s][3], &kk[4 * t],
                                                 &lam[4 * t], k_small, e.mult, e.shift);
        if constexpr (XP) {
          static_assert(!XP || TN == 4, "output tile rows are written 16 bytes at a time");
          *(v4i *)(ob + (16 * s + l16) * OROW + cb) = (v4i){(int)packed[0], (int)packed[1 % TN], (int)packed[2 % TN], (int)packed[3 % TN]};
        } else {
          // Every lane stores, without a branch: lanes past the last pixel of the run hold
          // the results of that pixel (their loads were clamped to it) and rewrite them.
          const int m = min(p0 + 16 * s + l16, px_end - 1);
          uint8_t *o = (uint8_t *)g.out + (long long)m * N + cb;
          if constexpr (TN == 4) store16<NT>(o, (v4i){(int)packed[0], (int)packed[1 % TN], (int)packed[2 % TN], (int)packed[3 % TN]});
          else if constexpr (TN == 2) store8<NT>(o, (v2i){(int)packed[0], (int)packed[1 % TN]});
          else store4<NT>(o, (int)packed[0]);
        }
      }
    }
    if constexpr (XP) {
      // The tile in memory order: piece idx = r*64 + lane is bytes [16*idx, 16*idx + 16) of the
      // step's PX * N contiguous output bytes.  Rows past the end of the run are redirected
      // to its last row (same bytes to the same address): no branch, fixed store count.
      constexpr int CPR = N / 16, NR = PX * N / 1024;
      const int last = px_end - 1 - p0;
      v4i v[NR];
      long long go[NR];
#pragma unroll
      for (int r = 0; r < NR; r++) {
        const int idx = r * 64 + lane, row = min(idx / CPR, last), col = (idx % CPR) * 16;
        v[r] = *(const v4i *)(ob + row * OROW + col);
        go[r] = (long long)(p0 + row) * N + col;
      }
#pragma unroll
      for (int r = 0; r < NR; r++) store16<NT>((uint8_t *)g.out + go[r], v[r]);
    }
  };

  // Three register sets: the loads of step i+2 are issued, unconditionally (clamped to the
  // end of the run), before step i is computed.  The sets are handed down by register
  // moves in a single-copy loop body: the compiler derives how long a load may stay in
  // flight from the instructions issued behind it, and an unrolled rotation makes it merge
  // three different histories at the loop header into a wait for everything.
  auto stream = [&](auto nt) {
    for (; px < px_end; px += PX) {
      load_a(b2, px + 2 * PX);
      process(b0, px, nt);
#pragma unroll
      for (int s = 0; s < TM; s++)
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          b0[s][ks] = b1[s][ks];
          b1[s][ks] = b2[s][ks];
        }
    }
  };
  // the store policy is fixed per launch: one copy of the loop for each, no branch per store
  if (g.nt) stream(std::true_type{});
  else stream(std::false_type{});
}
