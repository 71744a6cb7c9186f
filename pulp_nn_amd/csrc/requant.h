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

// ---- packed fast paths --------------------------------------------------------
// v_ashr_pk_u8_i32 d, a, b, s: d[7:0] = sat_u8(a >> s[4:0]), d[15:8] = sat_u8(b >> s[4:0]);
// with op_sel:[0,0,0,1] the two bytes go to d[31:16] instead; the other half of d is
// left as it was (measured on gfx950).  Issued through inline asm because hipcc 7.2
// models the instruction as clearing the other half.
// The inputs of this version must come from ordinary VALU instructions, not straight
// from MFMA accumulators: the compiler does not insert the MFMA -> VALU wait states in
// front of inline asm.
__device__ __forceinline__ unsigned ashr_sat_pack4(int a0, int a1, int a2, int a3, int shift)
{
  unsigned d;
  asm("v_ashr_pk_u8_i32 %0, %1, %2, %3" : "=v"(d) : "v"(a0), "v"(a1), "v"(shift));
  asm("v_ashr_pk_u8_i32 %0, %1, %2, %3 op_sel:[0,0,0,1]" : "+v"(d) : "v"(a2), "v"(a3), "v"(shift));
  return d;
}

// Same result through the compiler's own builtin (safe directly after MFMA, three
// instructions more: the builtin's 16-bit results are masked before the byte merge).
__device__ __forceinline__ unsigned ashr_sat_pack4_safe(int a0, int a1, int a2, int a3, int shift)
{
  const unsigned lo = __builtin_amdgcn_ashr_pk_u8_i32(a0, a1, shift);
  const unsigned hi = __builtin_amdgcn_ashr_pk_u8_i32(a2, a3, shift);
  return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

// Requantise four accumulators (four consecutive channels, parameters k[0..3],
// lambda[0..3]) into four packed bytes.  ACC24 promises |acc| < 2^23, which lets
// the 32-bit products use the full-rate 24-bit multiplier (the low 32 bits of the
// 48-bit product are exactly the wrapped 32-bit product).  k24 says that the four
// k values fit 24 bits (32-bit build) or 32 bits (64-bit build) as signed numbers.
// WIDE (multiplier branch only) promises shift >= 16: prod >> shift then already
// fits int16_t, so the reference's narrowing to int16_t changes nothing.
template <int MODE, bool ACC24, bool WIDE = false>
__device__ __forceinline__ unsigned requant4(int a0, int a1, int a2, int a3, const bn_t *k, const bn_t *lambda,
                                             bool k_small, int mult, int shift)
{
  if constexpr (MODE == EPI_RAW) {
    return ashr_sat_pack4_safe(a0, a1, a2, a3, shift);
  } else if constexpr (MODE == EPI_MULT) {
    int p0, p1, p2, p3;
    if constexpr (ACC24) {
      p0 = __mul24(a0, mult);
      p1 = __mul24(a1, mult);
      p2 = __mul24(a2, mult);
      p3 = __mul24(a3, mult);
    } else {
      p0 = (int)((unsigned)a0 * (unsigned)mult);
      p1 = (int)((unsigned)a1 * (unsigned)mult);
      p2 = (int)((unsigned)a2 * (unsigned)mult);
      p3 = (int)((unsigned)a3 * (unsigned)mult);
    }
    if constexpr (WIDE) return ashr_sat_pack4(p0, p1, p2, p3, shift);
    // (int16_t)(prod >> shift), then clamp
    p0 = (int)(short)(p0 >> shift);
    p1 = (int)(short)(p1 >> shift);
    p2 = (int)(short)(p2 >> shift);
    p3 = (int)(short)(p3 >> shift);
    return ashr_sat_pack4(p0, p1, p2, p3, 0);
  } else {
#if PULPNN_BN_BITS == 64
    if (k_small) {
      // 32 x 32 -> 64 bit multiply-add, then the low 32 bits of the 64-bit arithmetic shift
      long long v0 = (long long)(int)k[0] * (long long)a0 + lambda[0];
      long long v1 = (long long)(int)k[1] * (long long)a1 + lambda[1];
      long long v2 = (long long)(int)k[2] * (long long)a2 + lambda[2];
      long long v3 = (long long)(int)k[3] * (long long)a3 + lambda[3];
      int x0, x1, x2, x3;
      if (shift >= 32) {
        x0 = (int)(v0 >> 32);
        x1 = (int)(v1 >> 32);
        x2 = (int)(v2 >> 32);
        x3 = (int)(v3 >> 32);
        return ashr_sat_pack4(x0, x1, x2, x3, shift - 32);
      }
      x0 = (int)__builtin_amdgcn_alignbit((unsigned)(v0 >> 32), (unsigned)v0, shift);
      x1 = (int)__builtin_amdgcn_alignbit((unsigned)(v1 >> 32), (unsigned)v1, shift);
      x2 = (int)__builtin_amdgcn_alignbit((unsigned)(v2 >> 32), (unsigned)v2, shift);
      x3 = (int)__builtin_amdgcn_alignbit((unsigned)(v3 >> 32), (unsigned)v3, shift);
      return ashr_sat_pack4(x0, x1, x2, x3, 0);
    }
    return (unsigned)requant<EPI_BN>(a0, k[0], lambda[0], mult, shift) |
           ((unsigned)requant<EPI_BN>(a1, k[1], lambda[1], mult, shift) << 8) |
           ((unsigned)requant<EPI_BN>(a2, k[2], lambda[2], mult, shift) << 16) |
           ((unsigned)requant<EPI_BN>(a3, k[3], lambda[3], mult, shift) << 24);
#else
    int v0, v1, v2, v3;
    if (ACC24 && k_small) {
      v0 = __mul24(a0, (int)k[0]) + (int)lambda[0];
      v1 = __mul24(a1, (int)k[1]) + (int)lambda[1];
      v2 = __mul24(a2, (int)k[2]) + (int)lambda[2];
      v3 = __mul24(a3, (int)k[3]) + (int)lambda[3];
    } else {
      v0 = (int)((unsigned)k[0] * (unsigned)a0 + (unsigned)lambda[0]);
      v1 = (int)((unsigned)k[1] * (unsigned)a1 + (unsigned)lambda[1]);
      v2 = (int)((unsigned)k[2] * (unsigned)a2 + (unsigned)lambda[2]);
      v3 = (int)((unsigned)k[3] * (unsigned)a3 + (unsigned)lambda[3]);
    }
    return ashr_sat_pack4(v0, v1, v2, v3, shift);
#endif
  }
}

// true when k is representable in 24 bits (32-bit build) / 32 bits (64-bit build)
__device__ __forceinline__ bool bn_k_small(bn_t k)
{
#if PULPNN_BN_BITS == 64
  return k == (bn_t)(int)k;
#else
  return k >= -(1 << 23) && k < (1 << 23);
#endif
}

// Four outputs of ONE channel (depthwise); |acc| < 2^23.  The accumulators come from
// v_dot4 instructions, so everything that reads them directly is compiler-visible code
// (the inline-asm pack only ever sees results of ordinary VALU instructions).
// FASTQ: batch-norm branch: k fits 24 bits (32-bit build) / 32 bits (64-bit build);
//        multiplier branch: shift >= 16 (the int16 narrowing is then the identity).
template <int MODE, bool FASTQ>
__device__ __forceinline__ unsigned requant4_same(int a0, int a1, int a2, int a3, bn_t k, bn_t lambda, int mult,
                                                  int shift)
{
  if constexpr (MODE == EPI_RAW) {
    return ashr_sat_pack4_safe(a0, a1, a2, a3, shift);
  } else if constexpr (MODE == EPI_MULT) {
    int p0 = __mul24(a0, mult), p1 = __mul24(a1, mult), p2 = __mul24(a2, mult), p3 = __mul24(a3, mult);
    if constexpr (FASTQ) return ashr_sat_pack4(p0, p1, p2, p3, shift);
    p0 = (int)(short)(p0 >> shift);
    p1 = (int)(short)(p1 >> shift);
    p2 = (int)(short)(p2 >> shift);
    p3 = (int)(short)(p3 >> shift);
    return ashr_sat_pack4(p0, p1, p2, p3, 0);
  } else {
#if PULPNN_BN_BITS == 64
    const bn_t kk[4] = {k, k, k, k}, ll[4] = {lambda, lambda, lambda, lambda};
    return requant4<EPI_BN, true>(a0, a1, a2, a3, kk, ll, FASTQ, mult, shift);
#else
    int v0, v1, v2, v3;
    if constexpr (FASTQ) {
      // compiler-visible multiplies: the accumulators come from v_dot4, whose results
      // other VALU instructions may only read after wait states the compiler inserts
      const int k32 = (int)k, l32 = (int)lambda;
      v0 = __mul24(a0, k32) + l32;
      v1 = __mul24(a1, k32) + l32;
      v2 = __mul24(a2, k32) + l32;
      v3 = __mul24(a3, k32) + l32;
    } else {
      v0 = (int)((unsigned)k * (unsigned)a0 + (unsigned)lambda);
      v1 = (int)((unsigned)k * (unsigned)a1 + (unsigned)lambda);
      v2 = (int)((unsigned)k * (unsigned)a2 + (unsigned)lambda);
      v3 = (int)((unsigned)k * (unsigned)a3 + (unsigned)lambda);
    }
    return ashr_sat_pack4(v0, v1, v2, v3, shift);
#endif
  }
}
