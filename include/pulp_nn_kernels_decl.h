/*
 * pulp_nn_kernels_decl.h -- the PULP-NN layer API on MI355X.
 *
 * Do not include directly: include 32bit/pulp_nn_kernels.h or
 * 64bit/pulp_nn_kernels.h, which set PULP_NN_BN_T (the type of the batch-norm
 * parameters k and lambda) to int32_t or int64_t, like the reference's two
 * trees, and link libpulpnn_hip32.so or libpulpnn_hip64.so respectively.
 *
 * Every function has the name, argument order and argument meaning of the
 * reference prototype cited next to it ({32bit,64bit}/include/pulp_nn_kernels.h).
 * Differences, all forced by the move to a GPU:
 *   - every pointer is a DEVICE pointer;
 *   - a call processes pulp_nn_hip_set_batch() images stored back to back and
 *     returns once the work is queued on pulp_nn_hip_set_stream()'s stream;
 *   - scratch arguments (pIm2ColBuffer, bufferC, bufferB, memory_chan) are
 *     accepted and ignored and may be NULL;
 *   - the _Ho_ / _HoWo_ / _Co_ variants, which differ only in how the reference
 *     splits work over its 8 cores, run the same kernel;
 *   - pulp_nn_maxpool leaves Im_in intact (the reference pools along x in place);
 *   - invalid arguments queue nothing and are reported through
 *     pulp_nn_hip_last_error() (the reference has no error channel).
 */
#ifndef PULP_NN_BN_T
#error "include 32bit/pulp_nn_kernels.h or 64bit/pulp_nn_kernels.h"
#endif

#include <stdint.h>
#include "pulp_nn_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Argument list shared by the three standard and three pointwise convolutions.
 * Note the order: x before y for sizes and strides, top/bottom before
 * left/right for padding. */
#define PULP_NN_CONV_ARGS                                                         \
  const uint8_t *pInBuffer, uint8_t *pIm2ColBuffer, const int8_t *bias,           \
  uint8_t *pOutBuffer, const int8_t *pWeight, PULP_NN_BN_T *k,                    \
  PULP_NN_BN_T *lambda, const uint16_t out_mult, const uint16_t out_shift,        \
  const uint16_t dim_in_x, const uint16_t dim_in_y, const uint16_t ch_in,         \
  const uint16_t dim_out_x, const uint16_t dim_out_y, const uint16_t ch_out,      \
  const uint16_t dim_kernel_x, const uint16_t dim_kernel_y,                       \
  const uint16_t padding_y_top, const uint16_t padding_y_bottom,                  \
  const uint16_t padding_x_left, const uint16_t padding_x_right,                  \
  const uint16_t stride_x, const uint16_t stride_y, int flag_relu,                \
  int flag_batch_norm

/* Standard convolution, HWC uint8 in/out, OHWI int8 weights, int8 bias.
 * Replaces pulp_nn_kernels.h:56-82, :84-110, :112-138. */
void pulp_nn_conv_Ho_parallel(PULP_NN_CONV_ARGS);
void pulp_nn_conv_Co_parallel(PULP_NN_CONV_ARGS);
void pulp_nn_conv_HoWo_parallel(PULP_NN_CONV_ARGS);

/* Pointwise (1x1) convolution; stride, padding and kernel-size arguments are
 * ignored exactly as in the reference.  Replaces pulp_nn_kernels.h:140-166,
 * :168-194, :196-222. */
void pulp_nn_pointwise_HoWo_parallel(PULP_NN_CONV_ARGS);
void pulp_nn_pointwise_Ho_parallel(PULP_NN_CONV_ARGS);
void pulp_nn_pointwise_Co_parallel(PULP_NN_CONV_ARGS);

/* Fully connected layer with uint8 output.  Replaces pulp_nn_kernels.h:224-237. */
void pulp_nn_linear(uint8_t *pInBuffer, int8_t *bias, uint8_t *pOutBuffer, int8_t *pWeights,
                    PULP_NN_BN_T *k, PULP_NN_BN_T *lambda, uint16_t out_mult, int8_t out_shift,
                    uint16_t dim_vec, uint16_t num_o_neurons, int flag_relu, int flag_batch_norm);

/* Fully connected layer with raw int32 output; bias points to int32 values.
 * Replaces pulp_nn_kernels.h:239-246. */
void pulp_nn_linear_out_32(uint8_t *pInBuffer, int8_t *bias, int32_t *pOutBuffer, int8_t *pWeights,
                           uint16_t dim_vec, uint16_t num_o_neurons);

/* The reference's inner two-pixel matmul: pInBuffer holds two columns of
 * num_col_im2col bytes; channel c of the first goes to pOut[c], of the second
 * to pOut2[c]; returns pOut + 2*ch_out like the reference.  Ignores the batch
 * count.  Replaces pulp_nn_kernels.h:248-262. */
uint8_t *pulp_nn_matmul(const int8_t *pWeight, uint8_t *pInBuffer, uint16_t ch_out, uint16_t num_col_im2col,
                        uint16_t out_shift, uint16_t out_mult, PULP_NN_BN_T *k, PULP_NN_BN_T *lambda,
                        const int8_t *bias, uint8_t *pOut, uint8_t *pOut2, int flag_relu, int flag_batch_norm);

/* Max pooling, HWC.  Replaces pulp_nn_kernels.h:264-280. */
void pulp_nn_maxpool(uint8_t *Im_in, uint8_t *Im_out, uint16_t dim_im_in_x, uint16_t dim_im_in_y,
                     uint16_t ch_im_in, uint16_t dim_im_out_x, uint16_t dim_im_out_y,
                     uint16_t dim_kernel_x, uint16_t dim_kernel_y, uint16_t padding_t, uint16_t padding_b,
                     uint16_t padding_l, uint16_t padding_r, uint16_t stride_x, uint16_t stride_y);

/* Average pooling with optional requantisation, HWC.  Replaces
 * pulp_nn_kernels.h:33-53 (lambda / out_add are int64_t in the 64bit tree). */
void pulp_nn_avgpool(uint8_t *Im_in, uint8_t *Im_out, PULP_NN_BN_T lambda, uint16_t out_shift,
                     PULP_NN_BN_T out_add, uint16_t dim_im_in_x, uint16_t dim_im_in_y, uint16_t ch_im_in,
                     uint16_t dim_im_out_x, uint16_t dim_im_out_y, uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                     uint16_t padding_t, uint16_t padding_b, uint16_t padding_l, uint16_t padding_r,
                     uint16_t stride_x, uint16_t stride_y, int flag_requant);

/* Element-wise requantised add.  Replaces pulp_nn_kernels.h:21-31. */
void pulp_nn_add(uint8_t *Im_in_1, uint8_t *Im_in_2, uint8_t *Im_out, uint16_t out_mult1, uint16_t out_mult2,
                 uint16_t out_shift, uint16_t dim_im_in_h, uint16_t dim_im_in_w, uint16_t ch_im_in);

/* Depthwise convolution, CHW uint8 in, [ch][ky][kx] int8 weights, HWC out.
 * Replaces pulp_nn_kernels.h:282-309 and :311-338. */
#define PULP_NN_DW_ARGS                                                           \
  const uint8_t *Im_in, uint8_t *bufferC, const int8_t *bias, uint8_t *Im_out,    \
  const int8_t *wt, uint8_t *bufferB, PULP_NN_BN_T *k, PULP_NN_BN_T *lambda,      \
  uint16_t out_mult, uint16_t out_shift, const uint16_t dim_im_in_x,              \
  const uint16_t dim_im_in_y, const uint16_t ch_im_in,                            \
  const uint16_t dim_im_out_x, const uint16_t dim_im_out_y,                       \
  const uint16_t ch_im_out, const uint16_t dim_kernel_x,                          \
  const uint16_t dim_kernel_y, const uint16_t padding_y_top,                      \
  const uint16_t padding_y_bottom, const uint16_t padding_x_left,                 \
  const uint16_t padding_x_right, const uint16_t stride_x,                        \
  const uint16_t stride_y, int8_t FLAG_RELU, int8_t FLAG_BATCH_NORM
void pulp_nn_depthwise_generic(PULP_NN_DW_ARGS);
void pulp_nn_depthwise_generic_less_4_weights(PULP_NN_DW_ARGS);

/* 3x3 stride-1 depthwise on a plane whose zero rows the caller has already
 * added (R = rows incl. padding, output has R-2 rows); no bias.  Only
 * p_l = p_r = 1 with even C is accepted: for any other combination the
 * reference's row pointers drift (pulp_nn_depthwise_3x3_s1.c:141-223).
 * Replaces pulp_nn_kernels.h:340-356. */
void pulp_nn_depthwise_3x3_s1(uint8_t *In_Img, uint8_t *Out_Img, int R, int C, int CH, int p_l, int p_r,
                              int8_t *Kernel, int8_t out_shift, uint16_t out_mult, PULP_NN_BN_T *kappa,
                              PULP_NN_BN_T *lambda, int flag_relu, int flag_batch_norm,
                              unsigned int *memory_chan);

#ifdef __cplusplus
}
#endif
