// Direct convolution for layers whose whole filter is at most 32 bytes long
// (K = ky * kx * Ci <= 32) and that have at most 32 output channels: the stem of
// a network (3x3 on RGB, 27 bytes per output channel).
//
// Such a layer is pure streaming (a few hundred multiply-adds per pixel against
// tens of bytes moved) and a GEMM tile is mostly padding for it, so it is done
// with v_dot4 on the vector ALUs instead: one output pixel per lane, its K input
// bytes gathered into 8 dwords (bytes past K and taps outside the image as zero),
// all weights and per-channel constants broadcast from LDS, the NCH results of a
// pixel packed and written as 16-byte pieces, one contiguous run per wave.
//
// Arithmetic as in igemm.h: activations as a ^ 0x80 with bias + 128 * sum_k w
// added back; exact in wrapping 32-bit arithmetic.
// Reference semantics: 32bit/src/pulp_nn_conv_Ho_parallel.c:76-183 (im2col order
// ky, kx, ci) and pulp_nn_matmul.c:144-216 (requantisation).
#pragma once
#include <type_traits>

#include "igemm.h"
#include "memops.h"
#include "requant.h"

#define SMALLK_KD 8  // filter dwords per channel (K <= 32)

template <int NCH, int MODE>
__global__ __launch_bounds__(256) void smallk_conv_kernel(ConvGeom g, EpiArgs e)
{
  __shared__ __attribute__((aligned(16))) int wl[NCH * SMALLK_KD];  // [channel][dword]
  __shared__ int corr_l[NCH];
  __shared__ bn_t k_l[NCH], lam_l[NCH];

  const int tid = threadIdx.x;
  // ---- weights and constants -> LDS -------------------------------------------------
  for (int q = tid; q < NCH * SMALLK_KD; q += 256) {
    const int n = q / SMALLK_KD, d = q % SMALLK_KD;
    unsigned v = 0;
    if (n < g.N) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int kk = 4 * d + j;
        if (kk < g.K) v |= (unsigned)(uint8_t)g.w[(long long)n * g.K + kk] << (8 * j);
      }
    }
    wl[q] = (int)v;
  }
  __syncthreads();
  if (tid < NCH) {
    int sum = 0;
#pragma unroll
    for (int d = 0; d < SMALLK_KD; d++) sum = __builtin_amdgcn_sdot4(wl[tid * SMALLK_KD + d], 0x01010101, sum, false);
    const bool real = tid < g.N;
    corr_l[tid] = 128 * sum + ((real && g.bias) ? (int)g.bias[tid] : 0);
    if (MODE == EPI_BN) {
      k_l[tid] = real ? e.k[tid] : 0;
      lam_l[tid] = real ? e.lambda[tid] : 0;
    }
  }
  __syncthreads();

  // ---- this lane's pixel: gather its K bytes -------------------------------------------
  const int m = blockIdx.x * 256 + tid;
  if (m >= g.M) return;
  const int b = m / g.HoWo, rem = m - b * g.HoWo;
  const int oy = rem / g.Wo, ox = rem - oy * g.Wo;
  const int iy0 = oy * g.sy - g.pt, ix0 = ox * g.sx - g.pl;
  const uint8_t *img = g.in + (long long)b * g.in_img;
  unsigned a[SMALLK_KD];
#pragma unroll
  for (int d = 0; d < SMALLK_KD; d++) a[d] = 0;
  {
    int fy = 0, fx = 0, ci = 0;
#pragma unroll
    for (int j = 0; j < 4 * SMALLK_KD; j++) {
      if (j < g.K) {
        const int iy = iy0 + fy, ix = ix0 + fx;
        if ((unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W)
          a[j >> 2] |= (unsigned)img[((long long)iy * g.W + ix) * g.Ci + ci] << (8 * (j & 3));
      }
      if (++ci == g.Ci) {
        ci = 0;
        if (++fx == g.kx) { fx = 0; ++fy; }
      }
    }
  }
#pragma unroll
  for (int d = 0; d < SMALLK_KD; d++) a[d] ^= 0x80808080u;

  // ---- NCH dot products, requantise, store ----------------------------------------------
  unsigned packed[NCH / 4];
#pragma unroll
  for (int n4 = 0; n4 < NCH / 4; n4++) {
    int acc[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int n = 4 * n4 + r;
      acc[r] = corr_l[n];
      const v4i w0 = *(const v4i *)&wl[n * SMALLK_KD], w1 = *(const v4i *)&wl[n * SMALLK_KD + 4];
      acc[r] = __builtin_amdgcn_sdot4((int)a[0], w0.x, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[1], w0.y, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[2], w0.z, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[3], w0.w, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[4], w1.x, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[5], w1.y, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[6], w1.z, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[7], w1.w, acc[r], false);
    }
    unsigned p = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int n = 4 * n4 + r;
      const bn_t kk = (MODE == EPI_BN) ? k_l[n] : (bn_t)0, ll = (MODE == EPI_BN) ? lam_l[n] : (bn_t)0;
      p |= (unsigned)requant<MODE>(acc[r], kk, ll, e.mult, e.shift) << (8 * r);
    }
    packed[n4] = p;
  }
  uint8_t *o = (uint8_t *)g.out + (long long)m * g.N;
  if (g.vec_store) {
    // N == NCH and 16-byte aligned rows: one copy of the store code per cache policy
    auto put = [&](auto nt) {
      constexpr bool NT = decltype(nt)::value;
#pragma unroll
      for (int q = 0; q < NCH / 16; q++)
        store16<NT>(o + 16 * q, (v4i){(int)packed[4 * q], (int)packed[4 * q + 1], (int)packed[4 * q + 2], (int)packed[4 * q + 3]});
    };
    if (g.nt) put(std::true_type{});
    else put(std::false_type{});
  } else {
#pragma unroll
    for (int n = 0; n < NCH; n++)
      if (n < g.N) o[n] = (uint8_t)(packed[n >> 2] >> (8 * (n & 3)));
  }
}
