// Skinny GEMM for linear layers with few rows (batch <= 256): weights stream,
// activations stay.
//
// pulp_nn_linear / pulp_nn_linear_out_32 (32bit/src/pulp_nn_linear.c:58-108,
// pulp_nn_linear_out_32.c) at small batch are bound by reading the weight matrix
// once; a tiled GEMM with a barrier per 64-byte K slice spends its time on
// per-slice latency instead (16 sequential slices for K = 1024).  Here a
// workgroup of four waves owns 16 output neurons.  The waves split the work by
// blocks of 64 rows and, when there are fewer than four such blocks, by parts of
// K as well (when the neurons alone make too few workgroups for the machine, the row blocks go to
// separate workgroups and K is always split in four); a wave fetches the weight fragment (16 rows x 64 bytes) and the
// activation fragments (64 rows x 64 bytes, shared by all workgroups and therefore
// cache resident) of four K slices at a time straight from global memory in the
// MFMA operand layout - twenty loads in flight, no staging - and the partial sums
// of the K parts meet in LDS at the end.
//
// Arithmetic as in igemm.h: activations as a ^ 0x80 with bias + 128 * sum_k w
// added back.
#pragma once
#include "igemm.h"
#include "requant.h"

struct SkinnyGeom {
  const uint8_t *in;   // [M][K]
  const int8_t *w;     // [N][K]
  const int8_t *bias;  // int8 [N]; int32 [N] for EPI_OUT32; may be null
  void *out;           // [M][N] uint8, or int32 for EPI_OUT32
  int M, N, K;         // M <= 256, K % 16 == 0, 16-byte aligned rows
  int kparts;          // 4, 2 or 1 parts of K; a workgroup takes 4 / kparts blocks of 64 rows, gridDim.y the rest
};

template <int MODE>
__global__ __launch_bounds__(256) void linear_skinny_kernel(SkinnyGeom g, EpiArgs e)
{
  __shared__ v4i part[4][4][64];  // [wave][s][lane]: partial accumulators of the K parts
  __shared__ int wpart[4][64];    // partial weight-row sums
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, lgrp = lane >> 4;
  const int n0 = blockIdx.x * 16;  // this workgroup's 16 neurons
  const int KT = (g.K + 63) / 64;
  // block of 64 rows (blockIdx.y counts the row blocks that other workgroups of the same neurons take), part of K
  const int rb = blockIdx.y * (4 / g.kparts) + wave / g.kparts, kp = wave % g.kparts;
  const int mb = rb * 64;
  const int kt0 = KT * kp / g.kparts, kt1 = KT * (kp + 1) / g.kparts;
  const bool active = mb < g.M;

  // weight rows past N and K chunks past K are read from a valid address and zeroed
  const bool nok = n0 + l16 < g.N;
  const int8_t *wrow = g.w + (long long)min(n0 + l16, g.N - 1) * g.K + 16 * lgrp;
  const uint8_t *arow[4];
#pragma unroll
  for (int s = 0; s < 4; s++) arow[s] = g.in + (long long)min(mb + 16 * s + l16, g.M - 1) * g.K + 16 * lgrp;

  int wsum = 0;  // this lane's share of sum_k w[n0 + l16][k] over this wave's part of K
  v4i acc[4];
#pragma unroll
  for (int s = 0; s < 4; s++) acc[s] = (v4i){0, 0, 0, 0};
  if (active) {
    for (int kb = kt0; kb < kt1; kb += 4) {
      // four slices: all loads first
      v4i wf[4], af[4][4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int kt = min(kb + u, kt1 - 1);
        const int ko = (64 * kt + 16 * lgrp < g.K) ? 64 * kt : 0;
        wf[u] = *(const v4i *)(wrow + ko);
#pragma unroll
        for (int s = 0; s < 4; s++) af[u][s] = *(const v4i *)(arow[s] + ko);
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int kt = kb + u;
        const bool ok = kt < kt1 && nok && 64 * kt + 16 * lgrp < g.K;
        if (!ok) wf[u] = (v4i){0, 0, 0, 0};
        wsum = __builtin_amdgcn_sdot4(wf[u].x, 0x01010101, wsum, false);
        wsum = __builtin_amdgcn_sdot4(wf[u].y, 0x01010101, wsum, false);
        wsum = __builtin_amdgcn_sdot4(wf[u].z, 0x01010101, wsum, false);
        wsum = __builtin_amdgcn_sdot4(wf[u].w, 0x01010101, wsum, false);
#pragma unroll
        for (int s = 0; s < 4; s++)
          acc[s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[u], af[u][s] ^ (int)0x80808080, acc[s], 0, 0, 0);
      }
    }
  }
  // ---- the K parts of a block of rows meet in LDS ---------------------------------------
  if (g.kparts > 1) {
#pragma unroll
    for (int s = 0; s < 4; s++) part[wave][s][lane] = acc[s];
    wpart[wave][lane] = wsum;
    __syncthreads();
    if (kp == 0) {
      for (int q = 1; q < g.kparts; q++) {
#pragma unroll
        for (int s = 0; s < 4; s++) acc[s] += part[wave + q][s][lane];
        wsum += wpart[wave + q][lane];
      }
    }
  }
  if (kp != 0 || !active) return;

  // ---- epilogue ---------------------------------------------------------------------------
  // acc[s][r] = neuron n0 + 4*lgrp + r of row mb + 16*s + l16
  int ws = wsum;
  ws += __shfl_xor(ws, 16);
  ws += __shfl_xor(ws, 32);  // every lane: sum of weight row n0 + l16
  int corr[4];
  bn_t kk[4], ll[4];
  bool ks = true;
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int n = n0 + 4 * lgrp + r;
    corr[r] = 128 * __shfl(ws, 4 * lgrp + r);
    kk[r] = 0;
    ll[r] = 0;
    if (n < g.N) {
      if (g.bias) corr[r] += (MODE == EPI_OUT32) ? ((const int *)g.bias)[n] : (int)g.bias[n];
      if (MODE == EPI_BN) {
        kk[r] = e.k[n];
        ll[r] = e.lambda[n];
      }
    }
    ks = ks && bn_k_small(kk[r]);
  }
  const bool k_small = __all(ks);
  const bool acc24 = g.K <= 256;
  constexpr int QM = MODE == EPI_OUT32 ? EPI_RAW : MODE;
#pragma unroll
  for (int s = 0; s < 4; s++) {
    const int m = mb + 16 * s + l16;
    if (m >= g.M) continue;
    const int a0 = acc[s][0] + corr[0], a1 = acc[s][1] + corr[1], a2 = acc[s][2] + corr[2], a3 = acc[s][3] + corr[3];
    const int nb = n0 + 4 * lgrp;
    if constexpr (MODE == EPI_OUT32) {
      int *o = (int *)g.out + (long long)m * g.N + nb;
      const int v[4] = {a0, a1, a2, a3};
#pragma unroll
      for (int r = 0; r < 4; r++)
        if (nb + r < g.N) o[r] = v[r];
    } else {
      const unsigned p = acc24 ? requant4<QM, true>(a0, a1, a2, a3, kk, ll, k_small, e.mult, e.shift)
                               : requant4<QM, false>(a0, a1, a2, a3, kk, ll, k_small, e.mult, e.shift);
      uint8_t *o = (uint8_t *)g.out + (long long)m * g.N + nb;
      if (nb + 4 <= g.N && (g.N & 3) == 0) {
        *(unsigned *)o = p;
      } else {
#pragma unroll
        for (int r = 0; r < 4; r++)
          if (nb + r < g.N) o[r] = (uint8_t)(p >> (8 * r));
      }
    }
  }
}
