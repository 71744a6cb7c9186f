// Weights-stationary streaming kernel for pointwise convolutions whose weight
// matrix is small (K <= 256, N <= 256): the HBM-bound case
// (pulp_nn_pointwise_HoWo_parallel at 28x28x128 -> 256 moves 384 bytes per pixel
// for 65 kop, far below the machine balance of ~625 op/B).
//
// The whole weight matrix sits in LDS in MFMA fragment order for the lifetime of
// a (persistent) workgroup, together with the per-channel constants.  Every wave
// streams its own pixels, 64 per step: the activation bytes go from HBM straight
// into registers in the MFMA column-operand layout (lane = pixel l%16, 16-byte K
// chunk l/16) and each byte is loaded by exactly one wave; the next step is
// prefetched while the current one is multiplied against all channel groups,
// requantised and stored.  There is no barrier after the weights are in place
// and no im2col.
//
// Arithmetic is that of igemm.h: activations as a ^ 0x80 with 128 * sum_k w
// added back (by starting the accumulators at bias + 128 * sum_k w).
#pragma once
#include "igemm.h"
#include "requant.h"

struct PwGeom {
  const uint8_t *in;   // [M][K] pixels, K = Ci contiguous
  const int8_t *w;     // [N][K]
  const int8_t *bias;  // int8 [N] (int32 for EPI_OUT32) or null
  void *out;           // [M][N]
  int M, N, K;
  int npass;           // channel groups of 16*TN (N == npass * 16 * TN)
  int pgroups;         // ceil(M / (16*TM)) pixel groups
};

// LDS bytes: weights, then k and lambda (bn_t), then corr (int) per padded channel, then a flag.
static inline int pw_lds_bytes(int tn, int ks, int npass, bool bn)
{
  return npass * 16 * tn * (ks * 64 + 4 + (bn ? 2 * (int)sizeof(bn_t) : 0)) + 16;
}

template <int TN, int KS, int MODE, bool WIDE, int TM>
__global__ __launch_bounds__(256, TM == 2 ? 4 : 2) void pw_stream_kernel(PwGeom g, EpiArgs e)
{
  // N == NP * 16 * TN: every lane owns 4*TN real channels
  constexpr int PX = 16 * TM;  // pixels per step
  constexpr int CG = 16 * TN;  // channels per pass
  extern __shared__ __attribute__((aligned(16))) unsigned char pw_lds[];
  const int npad = g.npass * CG;
  int8_t *Wl = (int8_t *)pw_lds;
  bn_t *kl = (bn_t *)(pw_lds + npad * KS * 64);
  bn_t *ll_ = kl + ((MODE == EPI_BN) ? npad : 0);
  int *corr_l = (int *)(ll_ + ((MODE == EPI_BN) ? npad : 0));
  int *flag_l = corr_l + npad;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
  const int l16 = lane & 15, lgrp = lane >> 4;

  // ---- first pixels on their way before anything else ---------------------------
  const int nwaves = gridDim.x * 4;
  int pg = blockIdx.x * 4 + wave;
  // Unconditional loads from clamped addresses (no per-lane branches, so that all
  // loads of a step are issued back to back and nothing waits on them here):
  // pixels past the end re-read the last pixel (their results are never stored) and
  // K chunks past the end re-read chunk 0 (their weights are zero).
  auto load_a = [&](v4i (&a)[TM][KS], int pgi) {
#pragma unroll
    for (int s = 0; s < TM; s++) {
      const int m = min(pgi * PX + 16 * s + l16, g.M - 1);
      const uint8_t *row = g.in + (long long)m * g.K;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const int k = ks * 64 + lgrp * 16;
        a[s][ks] = *(const v4i *)(row + (k < g.K ? k : 0));
      }
    }
  };
  v4i cur[TM][KS], nxt[TM][KS];
  load_a(cur, min(pg, g.pgroups - 1));

  // ---- weights and per-channel constants -> LDS -----------------------------------
  for (int n = tid; n < npad; n += 256) corr_l[n] = 0;
  if (tid == 0) *flag_l = 1;
  __syncthreads();
  {
    const int rows = npad * KS;  // 64-byte rows
    bool small = true;
    // batches of 8 chunks per thread so that 8 loads are in flight before the first LDS write
    for (int q0 = tid; q0 < rows * 4; q0 += 256 * 8) {
      v4i v[8];
      int nn[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int q = q0 + 256 * u;
        const int R = q >> 2, c = q & 3;
        const int i = R & 15, t = (R >> 4) % TN, ks = (R / CG) % KS, p = R / (CG * KS);
        nn[u] = p * CG + (i >> 2) * (4 * TN) + 4 * t + (i & 3);
        const int k = ks * 64 + 16 * c;
        v[u] = (v4i){0, 0, 0, 0};
        if (q < rows * 4 && nn[u] < g.N && k < g.K) v[u] = *(const v4i *)(g.w + (long long)nn[u] * g.K + k);
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int q = q0 + 256 * u;
        if (q >= rows * 4) break;  // uniform across the wave: rows * 4 is a multiple of 64
        const int R = q >> 2, c = q & 3;
        *(v4i *)&Wl[lds_off(R, c)] = v[u];
        int part = __builtin_amdgcn_sdot4(v[u].x, 0x01010101, 0, false);
        part = __builtin_amdgcn_sdot4(v[u].y, 0x01010101, part, false);
        part = __builtin_amdgcn_sdot4(v[u].z, 0x01010101, part, false);
        part = __builtin_amdgcn_sdot4(v[u].w, 0x01010101, part, false);
        part += __shfl_xor(part, 1);
        part += __shfl_xor(part, 2);
        if (c == 0) atomicAdd(&corr_l[nn[u]], 128 * part);
      }
    }
    for (int n = tid; n < npad; n += 256) {
      int b = 0;
      if (n < g.N && g.bias) b = (MODE == EPI_OUT32) ? ((const int *)g.bias)[n] : (int)g.bias[n];
      if (b) atomicAdd(&corr_l[n], b);
      if (MODE == EPI_BN) {
        const bn_t kv = n < g.N ? e.k[n] : 0;
        kl[n] = kv;
        ll_[n] = n < g.N ? e.lambda[n] : 0;
        small = small && bn_k_small(kv);
      }
    }
    if (!small) *flag_l = 0;
  }
  __syncthreads();
  const bool k_small = *flag_l != 0;

  // ---- stream pixels ------------------------------------------------------------------
  // One step: 64 pixels against every channel group.
  auto process = [&](v4i (&a)[TM][KS], int pgi) {
#pragma unroll
    for (int s = 0; s < TM; s++)
#pragma unroll
      for (int ks = 0; ks < KS; ks++) a[s][ks] ^= (int)0x80808080;

#pragma unroll 1
    for (int p = 0; p < g.npass; p++) {
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

      if constexpr (MODE == EPI_OUT32) {
#pragma unroll
        for (int s = 0; s < TM; s++) {
          const int m = pgi * PX + 16 * s + l16;
          if (m >= g.M) continue;
          int *o = (int *)g.out + (long long)m * g.N + cb;
#pragma unroll
          for (int c = 0; c < 4 * TN; c++)
            if (cb + c < g.N) o[c] = acc[c >> 2][s][c & 3];
        }
      } else {
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
          const int m = pgi * PX + 16 * s + l16;
          unsigned packed[TN];
#pragma unroll
          for (int t = 0; t < TN; t++)
            packed[t] = requant4<MODE, true, WIDE>(acc[t][s][0], acc[t][s][1], acc[t][s][2], acc[t][s][3], &kk[4 * t],
                                                   &lam[4 * t], k_small, e.mult, e.shift);
          {
            // Every lane stores, without a branch: lanes past the last pixel hold the
            // results of the last pixel (their loads were clamped to it) and rewrite them.
            uint8_t *o = (uint8_t *)g.out + (long long)min(m, g.M - 1) * g.N + cb;
            if constexpr (TN == 4) *(uint4 *)o = make_uint4(packed[0], packed[1], packed[2], packed[3]);
            else if constexpr (TN == 2) *(uint2 *)o = make_uint2(packed[0], packed[1]);
            else *(unsigned *)o = packed[0];
          }
        }
      }
    }
  };

  // One step per iteration: the loads of the next step are issued first, unconditionally
  // (clamped to the last group) and into registers nothing else touches, so that the only
  // wait on them is the register hand-over at the bottom of the loop.
  for (; pg < g.pgroups; pg += nwaves) {
    load_a(nxt, min(pg + nwaves, g.pgroups - 1));
    process(cur, pg);
#pragma unroll
    for (int s = 0; s < TM; s++)
#pragma unroll
      for (int ks = 0; ks < KS; ks++) cur[s][ks] = nxt[s][ks];
  }
}
