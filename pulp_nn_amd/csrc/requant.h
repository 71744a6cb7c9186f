// Device-side requantisation epilogue shared by every kernel.
//
// Integer arithmetic only.  Each branch reproduces the C types of the function
// it replaces:
//   EPI_BN    pulp_nn_bn_quant_u8   32bit/src/pulp_nn_utils.c:35-45 (int32, wrapping)
//                                   64bit/src/pulp_nn_utils.c:35-45 (int64, then the
//                                   clip truncates the shifted value to its low 32 bits)
//   EPI_MULT  pulp_nn_quant_u8      32bit/src/pulp_nn_utils.c:148-156 (int16 multiplier,
//                                   32-bit wrapping product, int16 narrowing before the clip)
//   EPI_RAW   clip8(sum >> shift)   32bit/src/pulp_nn_matmul.c:198-215
// The library is built twice, with PULPNN_BN_BITS = 32 and 64, mirroring the
// reference's 32bit/ and 64bit/ trees.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef PULPNN_BN_BITS
#error "define PULPNN_BN_BITS to 32 or 64"
#endif

#if PULPNN_BN_BITS == 64
typedef int64_t bn_t;
#else
typedef int32_t bn_t;
#endif

enum { EPI_BN = 0, EPI_MULT = 1, EPI_RAW = 2 };

// Scalar (per launch) epilogue parameters.
struct EpiArgs {
  const bn_t *k;       // [channels], EPI_BN only
  const bn_t *lambda;  // [channels], EPI_BN only
  int mult;            // (int16_t)out_mult, EPI_MULT only
  int shift;           // already converted like the reference converts it
};

// The empty asm keeps hipcc from fusing ">> shift, clamp to [0, 255], pack two
// bytes" into v_ashr_pk_u8_i32: hipcc 7.2 assumes that instruction clears bits
// 31:16 of its destination, but the hardware leaves them as they were, so the
// fused form ORs stale bits into neighbouring bytes.
__device__ __forceinline__ int clipu8(int x)
{
  asm volatile("" : "+v"(x));
  return min(max(x, 0), 255);
}

template <int MODE>
__device__ __forceinline__ int requant(int acc, bn_t k, bn_t lambda, int mult, int shift)
{
  if (MODE == EPI_BN) {
#if PULPNN_BN_BITS == 64
    unsigned long long v = (unsigned long long)k * (unsigned long long)(long long)acc + (unsigned long long)lambda;
    long long x = (long long)v >> shift;
    return clipu8((int)(unsigned)(unsigned long long)x);
#else
    unsigned v = (unsigned)k * (unsigned)acc + (unsigned)lambda;
    return clipu8((int)v >> shift);
#endif
  } else if (MODE == EPI_MULT) {
    int prod = (int)((unsigned)mult * (unsigned)acc);
    return clipu8((int)(short)(prod >> shift));
  } else {
    return clipu8(acc >> shift);
  }
}

// Which branch the reference takes for a pair of flags
// (32bit/src/pulp_nn_matmul.c:144-216).  relu_truthy selects the variant in
// pulp_nn_depthwise_generic.c:167-178, which tests FLAG_RELU for truth.
static inline int epi_mode(int flag_relu, int flag_batch_norm, bool relu_truthy = false)
{
  if (flag_batch_norm && flag_relu) return EPI_BN;
  if (relu_truthy ? (flag_relu != 0) : (flag_relu == 1)) return EPI_MULT;
  return EPI_RAW;
}
