/*
 * pulpnn_oracle.h -- CPU restatement of PULP-NN's int8 kernel arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the parity checker and the timed
 * CPU baseline.  Nothing in the shipped HIP path may call it.
 *
 * Every function restates, in plain scalar C, what one function of the
 * reference computes when it runs on a single core (NUM_CORES == 1).  The
 * reference files are cited per function in pulpnn_oracle.c.
 *
 * Conventions shared by all functions:
 *   bn_bits   32 or 64: the width of k / lambda (the reference's 32bit/ and
 *             64bit/ trees).  k and lambda are passed as const void* and read
 *             as int32_t[] or int64_t[] accordingly.
 *   batch     number of images, stored back to back (image stride = one
 *             image's bytes); weights, bias, k, lambda are shared.
 *   nthreads  images are distributed over this many OpenMP threads.
 */
#ifndef PULPNN_ORACLE_H
#define PULPNN_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The three-branch requantisation epilogue, one value at a time. */
uint8_t oracle_bn_quant_u8(int32_t phi, int64_t k, int64_t lambda, int8_t d, int bn_bits);
uint8_t oracle_quant_u8(int32_t phi, int16_t m, int8_t d);
uint8_t oracle_add_quant_u8(uint8_t pix1, uint8_t pix2, int16_t m1, int16_t m2, int8_t d);
/* shift_is_int8: 1 for the kernels whose out_shift parameter is int8_t
 * (linear, depthwise_3x3_s1), 0 where it is uint16_t. relu_eq1: 1 where the
 * reference tests flag_relu == 1 for the multiplier branch, 0 where it tests
 * truthiness (depthwise_generic). */
uint8_t oracle_epilogue(int32_t acc, int64_t k, int64_t lambda, uint16_t out_mult,
                        int out_shift, int flag_relu, int flag_batch_norm,
                        int bn_bits, int relu_eq1);

/* Standard convolution (all three _parallel variants compute this). */
void oracle_conv(const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *w,
                 const void *k, const void *lambda, uint16_t out_mult, uint16_t out_shift,
                 uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch_in,
                 uint16_t dim_out_x, uint16_t dim_out_y, uint16_t ch_out,
                 uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                 uint16_t pad_top, uint16_t pad_bottom, uint16_t pad_left, uint16_t pad_right,
                 uint16_t stride_x, uint16_t stride_y,
                 int flag_relu, int flag_batch_norm,
                 int bn_bits, int batch, int nthreads);

/* Same contraction, accumulators only (bias + sum), for pinning the index
 * arithmetic independently of the epilogue. acc is int32[batch][oy][ox][co]. */
void oracle_conv_acc(const uint8_t *in, const int8_t *bias, int32_t *acc, const int8_t *w,
                     uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch_in,
                     uint16_t dim_out_x, uint16_t dim_out_y, uint16_t ch_out,
                     uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                     uint16_t pad_top, uint16_t pad_bottom, uint16_t pad_left, uint16_t pad_right,
                     uint16_t stride_x, uint16_t stride_y, int batch, int nthreads);

/* Pointwise convolution: stride / padding / kernel arguments do not exist
 * here because the reference ignores them. */
void oracle_pointwise(const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *w,
                      const void *k, const void *lambda, uint16_t out_mult, uint16_t out_shift,
                      uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch_in,
                      uint16_t dim_out_x, uint16_t dim_out_y, uint16_t ch_out,
                      int flag_relu, int flag_batch_norm,
                      int bn_bits, int batch, int nthreads);

/* The two-pixel matmul helper: returns the number of bytes pOut advanced. */
void oracle_matmul(const int8_t *w, const uint8_t *in2, uint16_t ch_out, uint16_t num_col_im2col,
                   uint16_t out_shift, uint16_t out_mult, const void *k, const void *lambda,
                   const int8_t *bias, uint8_t *out, uint8_t *out2,
                   int flag_relu, int flag_batch_norm, int bn_bits);

void oracle_depthwise_3x3_s1(const uint8_t *in, uint8_t *out, int R, int C, int CH,
                             int p_l, int p_r, const int8_t *kernel, int8_t out_shift,
                             uint16_t out_mult, const void *kappa, const void *lambda,
                             int flag_relu, int flag_batch_norm,
                             int bn_bits, int batch, int nthreads);

void oracle_depthwise_generic(const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *wt,
                              const void *k, const void *lambda, uint16_t out_mult, uint16_t out_shift,
                              uint16_t dim_in_x, uint16_t dim_in_y,
                              uint16_t dim_out_x, uint16_t dim_out_y, uint16_t ch,
                              uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                              uint16_t pad_top, uint16_t pad_bottom, uint16_t pad_left, uint16_t pad_right,
                              uint16_t stride_x, uint16_t stride_y,
                              int8_t flag_relu, int8_t flag_batch_norm,
                              int bn_bits, int batch, int nthreads);

void oracle_linear(const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *w,
                   const void *k, const void *lambda, uint16_t out_mult, int8_t out_shift,
                   uint16_t dim_vec, uint16_t num_o_neurons, int flag_relu, int flag_batch_norm,
                   int bn_bits, int batch, int nthreads);

void oracle_linear_out_32(const uint8_t *in, const int8_t *bias, int32_t *out, const int8_t *w,
                          uint16_t dim_vec, uint16_t num_o_neurons, int batch, int nthreads);

/* clobber != 0 also reproduces the reference's in-place x pass on `in`. */
void oracle_maxpool(uint8_t *in, uint8_t *out, uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch,
                    uint16_t dim_out_x, uint16_t dim_out_y, uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                    uint16_t pad_t, uint16_t pad_b, uint16_t pad_l, uint16_t pad_r,
                    uint16_t stride_x, uint16_t stride_y, int clobber, int batch, int nthreads);

void oracle_avgpool(const uint8_t *in, uint8_t *out, int64_t lambda, uint16_t out_shift, int64_t out_add,
                    uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch,
                    uint16_t dim_out_x, uint16_t dim_out_y, uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                    uint16_t pad_t, uint16_t pad_b, uint16_t pad_l, uint16_t pad_r,
                    uint16_t stride_x, uint16_t stride_y, int flag_requant,
                    int bn_bits, int batch, int nthreads);

void oracle_add(const uint8_t *in1, const uint8_t *in2, uint8_t *out,
                uint16_t out_mult1, uint16_t out_mult2, uint16_t out_shift,
                uint16_t dim_h, uint16_t dim_w, uint16_t ch, int batch, int nthreads);

#ifdef __cplusplus
}
#endif
#endif
