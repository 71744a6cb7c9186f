/*
 * pulpnn_oracle.c -- CPU restatement of PULP-NN's int8 kernel arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY: the parity checker and the timed CPU baseline.
 * The shipped HIP path never calls into this file.
 *
 * What is restated: the result of each reference kernel when it runs on one
 * core (NUM_CORES == 1, pi_core_id() == 0), i.e. the mathematics plus every
 * width / wrap / truncation rule of the integer epilogue.  What is not
 * restated: the per-core work split, the im2col scratch buffers and the
 * 4-byte SIMD blocking; none of them changes a result.
 *
 * Citations are to /root/reference/{32bit,64bit}/src unless stated otherwise.
 * Build with -fwrapv: the reference relies on two's-complement wrap of int32.
 *
 * Pinning status (see tests/test_oracle_*.py): every function below is checked
 * against independent closed forms (numpy/scipy cross-correlation, GEMV,
 * windowed max / mean), hand-computed known answers for every branch of the
 * epilogue, and cross-function invariants.  The reference itself cannot be
 * compiled in this environment (it needs the PULP SDK's pmsis.h and the
 * Xpulp compiler builtins), so there is no compiled-reference comparison.
 */
#include "pulpnn_oracle.h"

#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* __builtin_pulp_clipu_r(x, 255) / __builtin_pulp_clipu(x, 0, 255): the
 * argument is a 32-bit int. */
static inline uint8_t clipu8(int32_t x)
{
  return (uint8_t)(x <= 0 ? 0 : (x >= 255 ? 255 : x));
}

static inline int64_t read_bn(const void *p, int i, int bn_bits)
{
  return bn_bits == 64 ? ((const int64_t *)p)[i] : (int64_t)((const int32_t *)p)[i];
}

/* pulp_nn_bn_quant_u8:
 *   32bit/src/pulp_nn_utils.c:35-45  int32 product, sum and shift (wrapping)
 *   64bit/src/pulp_nn_utils.c:35-45  int64 product, sum and shift; the clip
 *                                    builtin takes an int, so the shifted
 *                                    value is truncated to its low 32 bits. */
uint8_t oracle_bn_quant_u8(int32_t phi, int64_t k, int64_t lambda, int8_t d, int bn_bits)
{
  if (bn_bits == 64) {
    uint64_t v = (uint64_t)k * (uint64_t)(int64_t)phi + (uint64_t)lambda;
    int64_t x = (int64_t)v >> d;
    return clipu8((int32_t)(uint32_t)(uint64_t)x);
  } else {
    uint32_t v = (uint32_t)(int32_t)k * (uint32_t)phi + (uint32_t)(int32_t)lambda;
    int32_t x = (int32_t)v >> d;
    return clipu8(x);
  }
}

/* pulp_nn_quant_u8, 32bit/src/pulp_nn_utils.c:148-156 (identical in 64bit/):
 * the multiplier arrives as int16_t, the product wraps in 32 bits and the
 * shifted value is narrowed to int16_t before the clip. */
uint8_t oracle_quant_u8(int32_t phi, int16_t m, int8_t d)
{
  int32_t prod = (int32_t)((uint32_t)(int32_t)m * (uint32_t)phi);
  int16_t x = (int16_t)(prod >> d);
  return clipu8((int32_t)x);
}

/* pulp_nn_add_quant_u8, 32bit/src/pulp_nn_utils.c:47-60: the weighted sum is
 * held in a uint32_t, shifted logically and narrowed to uint16_t. */
uint8_t oracle_add_quant_u8(uint8_t pix1, uint8_t pix2, int16_t m1, int16_t m2, int8_t d)
{
  uint32_t v = (uint32_t)((int32_t)pix1 * (int32_t)m1 + (int32_t)pix2 * (int32_t)m2);
  uint16_t x = (uint16_t)(v >> d);
  return clipu8((int32_t)x);
}

/* Branch selection of the epilogue, 32bit/src/pulp_nn_matmul.c:144-216:
 *   flag_batch_norm && flag_relu -> bn_quant
 *   else flag_relu == 1          -> quant (scalar multiplier)
 *   else                         -> clip(acc >> out_shift)
 * pulp_nn_depthwise_generic.c:167-178 tests FLAG_RELU for truth instead of
 * == 1 (relu_eq1 == 0).  The quantiser functions receive the shift as int8_t.
 */
uint8_t oracle_epilogue(int32_t acc, int64_t k, int64_t lambda, uint16_t out_mult,
                        int out_shift, int flag_relu, int flag_batch_norm,
                        int bn_bits, int relu_eq1)
{
  if (flag_batch_norm && flag_relu)
    return oracle_bn_quant_u8(acc, k, lambda, (int8_t)out_shift, bn_bits);
  if (relu_eq1 ? (flag_relu == 1) : (flag_relu != 0))
    return oracle_quant_u8(acc, (int16_t)out_mult, (int8_t)out_shift);
  return clipu8(acc >> out_shift);
}

static inline int32_t dot_u8s8(const uint8_t *a, const int8_t *b, int n, int32_t acc)
{
  for (int i = 0; i < n; i++)
    acc += (int32_t)a[i] * (int32_t)b[i];
  return acc;
}

/* Accumulator of one output pixel / channel of the standard convolution.
 * pulp_nn_conv_Ho_parallel.c:76-164 gathers the ky x kx x ch_in patch with
 * zeros for taps outside the image, in (ky, kx, ci) order, which is also the
 * order of one weight row (OHWI); pulp_nn_matmul.c:70-142 starts from
 * (int)bias[c] (0 if bias == NULL) and adds the products. */
static inline int32_t conv_acc_one(const uint8_t *img, const int8_t *wrow, int32_t acc,
                                   int oy, int ox, int W, int H, int Ci, int kx, int ky,
                                   int pt, int pl, int sx, int sy)
{
  int iy0 = oy * sy - pt, ix0 = ox * sx - pl;
  for (int fy = 0; fy < ky; fy++) {
    int iy = iy0 + fy;
    if (iy < 0 || iy >= H) continue;
    for (int fx = 0; fx < kx; fx++) {
      int ix = ix0 + fx;
      if (ix < 0 || ix >= W) continue;
      acc = dot_u8s8(img + ((size_t)iy * W + ix) * Ci, wrow + ((size_t)fy * kx + fx) * Ci, Ci, acc);
    }
  }
  return acc;
}

/* pulp_nn_conv_{Ho,HoWo,Co}_parallel.c (e.g. pulp_nn_conv_Ho_parallel.c:30-249) */
void oracle_conv(const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *w,
                 const void *k, const void *lambda, uint16_t out_mult, uint16_t out_shift,
                 uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch_in,
                 uint16_t dim_out_x, uint16_t dim_out_y, uint16_t ch_out,
                 uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                 uint16_t pad_top, uint16_t pad_bottom, uint16_t pad_left, uint16_t pad_right,
                 uint16_t stride_x, uint16_t stride_y,
                 int flag_relu, int flag_batch_norm,
                 int bn_bits, int batch, int nthreads)
{
  (void)pad_bottom; (void)pad_right;
  const size_t in_img = (size_t)dim_in_x * dim_in_y * ch_in;
  const size_t out_img = (size_t)dim_out_x * dim_out_y * ch_out;
  const size_t K = (size_t)dim_kernel_x * dim_kernel_y * ch_in;
  const int bn = flag_batch_norm && flag_relu;
  const long rows = (long)batch * dim_out_y;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long row = 0; row < rows; row++) {
    int b = (int)(row / dim_out_y), oy = (int)(row % dim_out_y);
    const uint8_t *img = in + b * in_img;
    uint8_t *o = out + b * out_img + (size_t)oy * dim_out_x * ch_out;
    for (int ox = 0; ox < dim_out_x; ox++)
      for (int co = 0; co < ch_out; co++) {
        int32_t acc = bias ? (int32_t)bias[co] : 0;
        acc = conv_acc_one(img, w + co * K, acc, oy, ox, dim_in_x, dim_in_y, ch_in,
                           dim_kernel_x, dim_kernel_y, pad_top, pad_left, stride_x, stride_y);
        o[(size_t)ox * ch_out + co] =
            oracle_epilogue(acc, bn ? read_bn(k, co, bn_bits) : 0, bn ? read_bn(lambda, co, bn_bits) : 0,
                            out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
      }
  }
}

void oracle_conv_acc(const uint8_t *in, const int8_t *bias, int32_t *acc_out, const int8_t *w,
                     uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch_in,
                     uint16_t dim_out_x, uint16_t dim_out_y, uint16_t ch_out,
                     uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                     uint16_t pad_top, uint16_t pad_bottom, uint16_t pad_left, uint16_t pad_right,
                     uint16_t stride_x, uint16_t stride_y, int batch, int nthreads)
{
  (void)pad_bottom; (void)pad_right;
  const size_t in_img = (size_t)dim_in_x * dim_in_y * ch_in;
  const size_t out_img = (size_t)dim_out_x * dim_out_y * ch_out;
  const size_t K = (size_t)dim_kernel_x * dim_kernel_y * ch_in;
  const long rows = (long)batch * dim_out_y;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long row = 0; row < rows; row++) {
    int b = (int)(row / dim_out_y), oy = (int)(row % dim_out_y);
    const uint8_t *img = in + b * in_img;
    int32_t *o = acc_out + b * out_img + (size_t)oy * dim_out_x * ch_out;
    for (int ox = 0; ox < dim_out_x; ox++)
      for (int co = 0; co < ch_out; co++) {
        int32_t acc = bias ? (int32_t)bias[co] : 0;
        o[(size_t)ox * ch_out + co] =
            conv_acc_one(img, w + co * K, acc, oy, ox, dim_in_x, dim_in_y, ch_in,
                         dim_kernel_x, dim_kernel_y, pad_top, pad_left, stride_x, stride_y);
      }
  }
}

/* pulp_nn_pointwise_{HoWo,Ho,Co}_parallel.c: the input pixel of output (y, x)
 * is pInBuffer + (x + y*dim_in_x)*ch_in (pulp_nn_pointwise_HoWo_parallel.c:103,
 * pulp_nn_pointwise_Ho_parallel.c:79); stride, padding and kernel size are
 * never read.  Accumulation and epilogue are pulp_nn_matmul's. */
void oracle_pointwise(const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *w,
                      const void *k, const void *lambda, uint16_t out_mult, uint16_t out_shift,
                      uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch_in,
                      uint16_t dim_out_x, uint16_t dim_out_y, uint16_t ch_out,
                      int flag_relu, int flag_batch_norm,
                      int bn_bits, int batch, int nthreads)
{
  const size_t in_img = (size_t)dim_in_x * dim_in_y * ch_in;
  const size_t out_img = (size_t)dim_out_x * dim_out_y * ch_out;
  const int bn = flag_batch_norm && flag_relu;
  const long rows = (long)batch * dim_out_y;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long row = 0; row < rows; row++) {
    int b = (int)(row / dim_out_y), oy = (int)(row % dim_out_y);
    const uint8_t *img = in + b * in_img;
    uint8_t *o = out + b * out_img + (size_t)oy * dim_out_x * ch_out;
    for (int ox = 0; ox < dim_out_x; ox++) {
      const uint8_t *px = img + ((size_t)ox + (size_t)oy * dim_in_x) * ch_in;
      for (int co = 0; co < ch_out; co++) {
        int32_t acc = dot_u8s8(px, w + (size_t)co * ch_in, ch_in, bias ? (int32_t)bias[co] : 0);
        o[(size_t)ox * ch_out + co] =
            oracle_epilogue(acc, bn ? read_bn(k, co, bn_bits) : 0, bn ? read_bn(lambda, co, bn_bits) : 0,
                            out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
      }
    }
  }
}

/* pulp_nn_matmul.c:27-298: two im2col columns (in2 and in2 + num_col_im2col)
 * against ch_out weight rows; channel c of column 0 goes to out[c], of
 * column 1 to out2[c]. */
void oracle_matmul(const int8_t *w, const uint8_t *in2, uint16_t ch_out, uint16_t num_col_im2col,
                   uint16_t out_shift, uint16_t out_mult, const void *k, const void *lambda,
                   const int8_t *bias, uint8_t *out, uint8_t *out2,
                   int flag_relu, int flag_batch_norm, int bn_bits)
{
  const int bn = flag_batch_norm && flag_relu;
  for (int c = 0; c < ch_out; c++) {
    int32_t b0 = bias ? (int32_t)bias[c] : 0;
    int32_t s0 = dot_u8s8(in2, w + (size_t)c * num_col_im2col, num_col_im2col, b0);
    int32_t s1 = dot_u8s8(in2 + num_col_im2col, w + (size_t)c * num_col_im2col, num_col_im2col, b0);
    int64_t kk = bn ? read_bn(k, c, bn_bits) : 0, ll = bn ? read_bn(lambda, c, bn_bits) : 0;
    out[c] = oracle_epilogue(s0, kk, ll, out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
    out2[c] = oracle_epilogue(s1, kk, ll, out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
  }
}

/* pulp_nn_depthwise_3x3_s1.c:28-227, restated with the reference's own
 * pointer walk because its behaviour off the intended domain follows from it.
 * Input is CHW with planes of R x C bytes (:79-81), weights are [ch][3][3]
 * (:83-85), output is HWC with R-2 rows of C pixels (:110,145-146); there is no
 * bias and out_shift is int8_t.  Per output row (:103-223):
 *   p_l: output column 0 = taps (K1,K2) on the two bytes at the walk position
 *        of each of the three rows (:93-96,107-139);
 *   then pairs of output columns c, c+1 for c = p_l, p_l+2, ... < C-p_r, each
 *        from the four bytes at the walk position, which then moves on by 2
 *        (:141-186);
 *   p_r: one more output column from taps (K0,K1) (:98-101,187-219);
 *   then the walk position moves on by 2 (:220-222).
 * The walk lands on the start of the next input row only for p_l = p_r = 1
 * and even C; that is the domain in which this equals a 3x3 cross-correlation
 * with one zero column on either side.  Reads past the end of `in` (the
 * reference over-reads up to two bytes, multiplied by zero coefficients) and
 * writes past the end of `out` (odd C) are skipped here. */
void oracle_depthwise_3x3_s1(const uint8_t *in, uint8_t *out, int R, int C, int CH,
                             int p_l, int p_r, const int8_t *kernel, int8_t out_shift,
                             uint16_t out_mult, const void *kappa, const void *lambda,
                             int flag_relu, int flag_batch_norm,
                             int bn_bits, int batch, int nthreads)
{
  const size_t in_img = (size_t)R * C * CH;
  const size_t out_img = (size_t)(R - 2) * C * CH;
  const int bn = flag_batch_norm && flag_relu;
  const long jobs = (long)batch * CH;
#define RD(off) ((size_t)(off) < in_img ? img[(off)] : 0)
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long job = 0; job < jobs; job++) {
    int b = (int)(job / CH), ch = (int)(job % CH);
    const uint8_t *img = in + b * in_img;
    uint8_t *oimg = out + b * out_img;
    const int8_t *kw = kernel + ch * 9;
    int64_t kk = bn ? read_bn(kappa, ch, bn_bits) : 0, ll = bn ? read_bn(lambda, ch, bn_bits) : 0;
    size_t pos = (size_t)ch * R * C; /* walk position of the first of the three rows */
    for (int r = 0; r < R - 2; r++) {
      int c = 0;
      if (p_l) {
        int32_t s = 0;
        for (int i = 0; i < 3; i++)
          s += (int32_t)RD(pos + (size_t)i * C) * kw[i * 3 + 1] + (int32_t)RD(pos + (size_t)i * C + 1) * kw[i * 3 + 2];
        size_t t = (size_t)r * C * CH + ch;
        if (t < out_img)
          oimg[t] = oracle_epilogue(s, kk, ll, out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
      }
      for (c = p_l; c < C - p_r; c += 2) {
        int32_t s0 = 0, s1 = 0;
        for (int i = 0; i < 3; i++)
          for (int j = 0; j < 3; j++) {
            s0 += (int32_t)RD(pos + (size_t)i * C + j) * kw[i * 3 + j];
            s1 += (int32_t)RD(pos + (size_t)i * C + j + 1) * kw[i * 3 + j];
          }
        size_t t0 = (size_t)r * C * CH + (size_t)c * CH + ch, t1 = t0 + CH;
        if (t0 < out_img)
          oimg[t0] = oracle_epilogue(s0, kk, ll, out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
        if (t1 < out_img)
          oimg[t1] = oracle_epilogue(s1, kk, ll, out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
        pos += 2;
      }
      if (p_r) {
        int32_t s = 0;
        for (int i = 0; i < 3; i++)
          s += (int32_t)RD(pos + (size_t)i * C) * kw[i * 3 + 0] + (int32_t)RD(pos + (size_t)i * C + 1) * kw[i * 3 + 1];
        size_t t = (size_t)r * C * CH + (size_t)c * CH + ch;
        if (t < out_img)
          oimg[t] = oracle_epilogue(s, kk, ll, out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
      }
      pos += 2;
    }
  }
#undef RD
}

/* pulp_nn_depthwise_generic.c:30-391 (and _less_4_weights.c, same results):
 * CHW input (:74), [ch][ky][kx] weights (:75), HWC output (:81,179); a column
 * strip of the zero-padded plane is built per output column (:82-132,185-229,
 * 281-336) and each output row is a ky*kx dot product on it starting from
 * (int)bias[ch] (:138-166).  k / lambda are indexed per channel (:167-169 with
 * :387-388).  The multiplier branch is taken for any non-zero FLAG_RELU. */
void oracle_depthwise_generic(const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *wt,
                              const void *k, const void *lambda, uint16_t out_mult, uint16_t out_shift,
                              uint16_t dim_in_x, uint16_t dim_in_y,
                              uint16_t dim_out_x, uint16_t dim_out_y, uint16_t ch,
                              uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                              uint16_t pad_top, uint16_t pad_bottom, uint16_t pad_left, uint16_t pad_right,
                              uint16_t stride_x, uint16_t stride_y,
                              int8_t flag_relu, int8_t flag_batch_norm,
                              int bn_bits, int batch, int nthreads)
{
  (void)pad_bottom; (void)pad_right;
  const size_t in_img = (size_t)dim_in_x * dim_in_y * ch;
  const size_t out_img = (size_t)dim_out_x * dim_out_y * ch;
  const int bn = flag_batch_norm && flag_relu;
  const long jobs = (long)batch * ch;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long job = 0; job < jobs; job++) {
    int b = (int)(job / ch), c = (int)(job % ch);
    const uint8_t *plane = in + b * in_img + (size_t)c * dim_in_x * dim_in_y;
    const int8_t *kw = wt + (size_t)c * dim_kernel_x * dim_kernel_y;
    int64_t kk = bn ? read_bn(k, c, bn_bits) : 0, ll = bn ? read_bn(lambda, c, bn_bits) : 0;
    uint8_t *o = out + b * out_img + c;
    for (int oy = 0; oy < dim_out_y; oy++)
      for (int ox = 0; ox < dim_out_x; ox++) {
        int32_t acc = bias ? (int32_t)bias[c] : 0;
        for (int fy = 0; fy < dim_kernel_y; fy++) {
          int iy = oy * stride_y - pad_top + fy;
          if (iy < 0 || iy >= dim_in_y) continue;
          for (int fx = 0; fx < dim_kernel_x; fx++) {
            int ix = ox * stride_x - pad_left + fx;
            if (ix < 0 || ix >= dim_in_x) continue;
            acc += (int32_t)plane[(size_t)iy * dim_in_x + ix] * (int32_t)kw[fy * dim_kernel_x + fx];
          }
        }
        o[((size_t)oy * dim_out_x + ox) * ch] =
            oracle_epilogue(acc, kk, ll, out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 0);
      }
  }
}

/* pulp_nn_linear.c:29-111: one GEMV per image; out_shift is int8_t. */
void oracle_linear(const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *w,
                   const void *k, const void *lambda, uint16_t out_mult, int8_t out_shift,
                   uint16_t dim_vec, uint16_t num_o_neurons, int flag_relu, int flag_batch_norm,
                   int bn_bits, int batch, int nthreads)
{
  const int bn = flag_batch_norm && flag_relu;
  const long jobs = (long)batch * num_o_neurons;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long job = 0; job < jobs; job++) {
    int b = (int)(job / num_o_neurons), n = (int)(job % num_o_neurons);
    int32_t acc = dot_u8s8(in + (size_t)b * dim_vec, w + (size_t)n * dim_vec, dim_vec,
                           bias ? (int32_t)bias[n] : 0);
    out[(size_t)b * num_o_neurons + n] =
        oracle_epilogue(acc, bn ? read_bn(k, n, bn_bits) : 0, bn ? read_bn(lambda, n, bn_bits) : 0,
                        out_mult, out_shift, flag_relu, flag_batch_norm, bn_bits, 1);
  }
}

/* pulp_nn_linear_out_32.c:28-82: the bias pointer is typed int8_t* but neuron
 * i reads a 32-bit value at byte offset 4*i (:52-55); the sum is stored
 * unquantised (:78). */
void oracle_linear_out_32(const uint8_t *in, const int8_t *bias, int32_t *out, const int8_t *w,
                          uint16_t dim_vec, uint16_t num_o_neurons, int batch, int nthreads)
{
  const long jobs = (long)batch * num_o_neurons;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long job = 0; job < jobs; job++) {
    int b = (int)(job / num_o_neurons), n = (int)(job % num_o_neurons);
    int32_t b32 = 0;
    if (bias) memcpy(&b32, bias + 4 * (size_t)n, 4);
    out[(size_t)b * num_o_neurons + n] =
        dot_u8s8(in + (size_t)b * dim_vec, w + (size_t)n * dim_vec, dim_vec, b32);
  }
}

/* pulp_nn_maxpool.c:27-146, restated pass by pass because the first pass
 * works in place on the input and the second reads what the first left:
 *   pass 1 (:58-94)  for every INPUT row and every output column i_x, the
 *       pixel at column i_x of that row becomes the unsigned per-channel max
 *       of columns [ws, we): ws = i_x*sx - pl, or i_x itself when that is
 *       negative; we = min(i_x*sx - pl + kx, W).
 *   pass 2 (:107-144) output row i_y is the max over input rows
 *       [max(i_y*sy - pt, 0), min(i_y*sy - pt + ky, H)) of the first
 *       dim_out_x pixels of each row.
 * With clobber == 0 the first pass runs on a private copy. */
void oracle_maxpool(uint8_t *in, uint8_t *out, uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch,
                    uint16_t dim_out_x, uint16_t dim_out_y, uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                    uint16_t pad_t, uint16_t pad_b, uint16_t pad_l, uint16_t pad_r,
                    uint16_t stride_x, uint16_t stride_y, int clobber, int batch, int nthreads)
{
  (void)pad_b; (void)pad_r;
  const size_t in_img = (size_t)dim_in_x * dim_in_y * ch;
  const size_t out_img = (size_t)dim_out_x * dim_out_y * ch;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (int b = 0; b < batch; b++) {
    uint8_t *img = in + b * in_img;
    uint8_t *work = img;
    if (!clobber) {
      work = (uint8_t *)malloc(in_img);
      memcpy(work, img, in_img);
    }
    for (int iy = 0; iy < dim_in_y; iy++)
      for (int ix = 0; ix < dim_out_x; ix++) {
        uint8_t *target = work + ((size_t)iy * dim_in_x + ix) * ch;
        int ws = ix * stride_x - pad_l;
        int we = ws + dim_kernel_x;
        if (ws < 0) ws = ix;
        if (we >= dim_in_x) we = dim_in_x;
        const uint8_t *src = work + ((size_t)iy * dim_in_x + ws) * ch;
        for (int c = 0; c < ch; c++) target[c] = src[c];
        for (int x = ws + 1; x < we; x++) {
          src = work + ((size_t)iy * dim_in_x + x) * ch;
          for (int c = 0; c < ch; c++)
            if (target[c] < src[c]) target[c] = src[c];
        }
      }
    for (int oy = 0; oy < dim_out_y; oy++) {
      uint8_t *target = out + b * out_img + (size_t)oy * dim_out_x * ch;
      int rs = oy * stride_y - pad_t;
      int re = rs + dim_kernel_y;
      if (rs < 0) rs = 0;
      if (re >= dim_in_y) re = dim_in_y;
      const size_t n = (size_t)dim_out_x * ch;
      const uint8_t *src = work + (size_t)rs * dim_in_x * ch;
      for (size_t i = 0; i < n; i++) target[i] = src[i];
      for (int y = rs + 1; y < re; y++) {
        src = work + (size_t)y * dim_in_x * ch;
        for (size_t i = 0; i < n; i++)
          if (target[i] < src[i]) target[i] = src[i];
      }
    }
    if (!clobber) free(work);
  }
}

/* pulp_nn_avgpool.c:29-121.  Window bounds as written there (:82-86): the
 * y start uses padding_b and the x end uses padding_r.  The divisor is always
 * kx*ky (:66).  Requantisation (:106-110): in the 32bit tree
 * (sum*lambda/ksize + out_add) >> out_shift is evaluated in uint32_t (sum is
 * uint32_t) and stored to an int32_t; in the 64bit tree (64bit/...:106) it is
 * int64_t arithmetic whose result the clip truncates to int. */
void oracle_avgpool(const uint8_t *in, uint8_t *out, int64_t lambda, uint16_t out_shift, int64_t out_add,
                    uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch,
                    uint16_t dim_out_x, uint16_t dim_out_y, uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                    uint16_t pad_t, uint16_t pad_b, uint16_t pad_l, uint16_t pad_r,
                    uint16_t stride_x, uint16_t stride_y, int flag_requant,
                    int bn_bits, int batch, int nthreads)
{
  const size_t in_img = (size_t)dim_in_x * dim_in_y * ch;
  const size_t out_img = (size_t)dim_out_x * dim_out_y * ch;
  const uint32_t ksize = (uint32_t)dim_kernel_x * dim_kernel_y;
  const long rows = (long)batch * dim_out_y;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long row = 0; row < rows; row++) {
    int b = (int)(row / dim_out_y), oy = (int)(row % dim_out_y);
    const uint8_t *img = in + b * in_img;
    for (int ox = 0; ox < dim_out_x; ox++) {
      int ys = oy * stride_y - pad_b; if (ys < 0) ys = 0;
      int ye = oy * stride_y - pad_t + dim_kernel_y; if (ye > dim_in_y) ye = dim_in_y;
      int xs = ox * stride_x - pad_l; if (xs < 0) xs = 0;
      int xe = ox * stride_x - pad_r + dim_kernel_x; if (xe > dim_in_x) xe = dim_in_x;
      uint8_t *o = out + b * out_img + ((size_t)oy * dim_out_x + ox) * ch;
      for (int c = 0; c < ch; c++) {
        uint32_t sum = 0;
        for (int y = ys; y < ye; y++)
          for (int x = xs; x < xe; x++)
            sum += img[((size_t)y * dim_in_x + x) * ch + c];
        int32_t res;
        if (flag_requant) {
          if (bn_bits == 64) {
            int64_t v = (int64_t)((uint64_t)sum * (uint64_t)lambda);
            v = v / (int64_t)ksize;
            v = (int64_t)((uint64_t)v + (uint64_t)out_add);
            res = (int32_t)(uint32_t)(uint64_t)(v >> out_shift);
          } else {
            uint32_t v = sum * (uint32_t)(int32_t)lambda / ksize + (uint32_t)(int32_t)out_add;
            res = (int32_t)(v >> out_shift);
          }
        } else {
          res = (int32_t)(sum / ksize);
        }
        o[c] = clipu8(res);
      }
    }
  }
}

/* pulp_nn_add.c:27-62 over H*W*C bytes with pulp_nn_add_quant_u8. */
void oracle_add(const uint8_t *in1, const uint8_t *in2, uint8_t *out,
                uint16_t out_mult1, uint16_t out_mult2, uint16_t out_shift,
                uint16_t dim_h, uint16_t dim_w, uint16_t ch, int batch, int nthreads)
{
  const long n = (long)batch * dim_h * dim_w * ch;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (long i = 0; i < n; i++)
    out[i] = oracle_add_quant_u8(in1[i], in2[i], (int16_t)out_mult1, (int16_t)out_mult2, (int8_t)out_shift);
}
