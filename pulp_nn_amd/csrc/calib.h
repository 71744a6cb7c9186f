// Calibration of out_shift: max |acc * k[c]| over a whole layer.
//
// A network that requantises with batch-norm picks, per layer,
// out_shift = floor(log2(max |acc * k|)) - 7, so that the largest product lands in the
// top of the uint8 range.  acc is the layer's accumulator including bias
// (32bit/src/pulp_nn_matmul.c:70-142 for conv / pointwise / linear,
// pulp_nn_depthwise_generic.c:138-166 for depthwise), 32-bit wrapping; the product is taken
// in 64-bit wrapping arithmetic like (int64_t)k * acc in the 64-bit tree.
//
// This is a one-off pass, not a hot path: one output per thread and a plain loop over the
// taps.  Each workgroup takes CALIB_CHUNK consecutive outputs and leaves the maximum of its
// chunk in partial[blockIdx.x] (a plain store: every slot that is read has been written by
// this launch, so the buffer needs no clearing); calib_final_kernel reduces the slots.
#pragma once
#include "requant.h"

#define CALIB_CHUNK 65536  // outputs per workgroup

struct CalibGeom {
  const uint8_t *in;
  const int8_t *w;
  const int8_t *bias;  // int8 [Co], may be null
  const bn_t *k;       // [Co]
  long long total;     // B * Ho * Wo * Co outputs
  long long in_img;    // bytes per input image
  int H, W, Ci, Ho, Wo, Co;
  int kx, ky, pt, pl, sx, sy;
  int depthwise;  // one filter [ky][kx] per channel, Ci == Co
  int chw_in;     // depthwise only: the input is CHW (else HWC)
};

__device__ __forceinline__ unsigned long long calib_mag(int acc, bn_t k)
{
  const unsigned long long v = (unsigned long long)(long long)k * (unsigned long long)(long long)acc;
  return ((long long)v < 0) ? (0ull - v) : v;
}

__global__ __launch_bounds__(256) void calib_absmax_kernel(CalibGeom g, unsigned long long *partial)
{
  __shared__ unsigned long long red[4];
  const long long first = (long long)blockIdx.x * CALIB_CHUNK;
  unsigned long long best = 0;
  for (int i = threadIdx.x; i < CALIB_CHUNK; i += 256) {
    const long long idx = first + i;
    if (idx >= g.total) break;
    const int co = (int)(idx % g.Co);
    long long m = idx / g.Co;
    const int ox = (int)(m % g.Wo);
    m /= g.Wo;
    const int oy = (int)(m % g.Ho);
    const long long b = m / g.Ho;
    const uint8_t *img = g.in + b * g.in_img;
    unsigned acc = g.bias ? (unsigned)(int)g.bias[co] : 0u;
    for (int fy = 0; fy < g.ky; fy++) {
      const int iy = oy * g.sy - g.pt + fy;
      if ((unsigned)iy >= (unsigned)g.H) continue;
      for (int fx = 0; fx < g.kx; fx++) {
        const int ix = ox * g.sx - g.pl + fx;
        if ((unsigned)ix >= (unsigned)g.W) continue;
        if (g.depthwise) {
          const int a = g.chw_in ? img[((long long)co * g.H + iy) * g.W + ix] : img[((long long)iy * g.W + ix) * g.Ci + co];
          acc += (unsigned)(a * (int)g.w[((long long)co * g.ky + fy) * g.kx + fx]);
        } else {
          const uint8_t *a = img + ((long long)iy * g.W + ix) * g.Ci;
          const int8_t *wr = g.w + (((long long)co * g.ky + fy) * g.kx + fx) * g.Ci;
          int s = 0;
          for (int ci = 0; ci < g.Ci; ci++) s += (int)a[ci] * (int)wr[ci];
          acc += (unsigned)s;
        }
      }
    }
    const unsigned long long v = calib_mag((int)acc, g.k[co]);
    best = v > best ? v : best;
  }
  // wave maximum, then the four waves through LDS
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned long long other = __shfl_xor(best, o);
    best = other > best ? other : best;
  }
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; w++) best = red[w] > best ? red[w] : best;
    partial[blockIdx.x] = best;
  }
}

// result[0] = max over the slots, result[1] = max(floor(log2(result[0])) - 7, 0) (0 for an all-zero layer)
__global__ __launch_bounds__(256) void calib_final_kernel(const unsigned long long *partial, int slots,
                                                          unsigned long long *result)
{
  __shared__ unsigned long long red[4];
  unsigned long long best = 0;
  for (int i = threadIdx.x; i < slots; i += 256) best = partial[i] > best ? partial[i] : best;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned long long other = __shfl_xor(best, o);
    best = other > best ? other : best;
  }
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; w++) best = red[w] > best ? red[w] : best;
    result[0] = best;
    const int lg = best ? 63 - __builtin_clzll(best) : 0;
    result[1] = (unsigned long long)(lg > 7 ? lg - 7 : 0);
  }
}
