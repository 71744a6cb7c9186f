/*
 * pulp_nn_hip.h -- entry points this library adds to the PULP-NN kernel API.
 *
 * The layer functions themselves keep the names and argument lists of the
 * reference's pulp_nn_kernels.h (see include/32bit and include/64bit); they
 * take DEVICE pointers and return as soon as the work is queued on the
 * library's stream.  Because those functions return void and the reference has
 * no batch dimension, no stream and no error channel, the calls below supply
 * them.  They have no counterpart in the reference.
 *
 * All state set here is per host thread.
 */
#ifndef PULP_NN_HIP_H
#define PULP_NN_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

enum {
  PULP_NN_HIP_OK = 0,
  PULP_NN_HIP_ERR_ARGUMENT = 1,     /* null pointer, zero dimension, shift out of range */
  PULP_NN_HIP_ERR_UNSUPPORTED = 2,  /* geometry outside what the reference itself handles */
  PULP_NN_HIP_ERR_RUNTIME = 3       /* a HIP call failed */
};

/* Number of images processed by every following layer call (default 1).
 * Images are stored back to back in every activation buffer: image i of a
 * tensor starts i * (bytes of one image) after the pointer passed to the layer
 * function.  Weights, bias, k and lambda are shared by all images. */
void pulp_nn_hip_set_batch(unsigned n_images);
unsigned pulp_nn_hip_get_batch(void);

/* hipStream_t (as void*) on which following layer calls are queued; NULL is
 * the default stream. */
void pulp_nn_hip_set_stream(void *hip_stream);
void *pulp_nn_hip_get_stream(void);

/* Wait for everything queued on the current stream.  Returns a status code. */
int pulp_nn_hip_sync(void);

/* Measurement aid (no counterpart in the reference): queues a one-wave kernel on the current stream that runs for
 * 20 us and writes two 64-bit counts to device memory: out[0] = ticks of the 100 MHz wall clock, out[1] = cycles of the
 * shader clock over the same interval (shader MHz = 100 * out[1] / out[0]).  Queued behind a run of layer calls it
 * tells at which clock the GPU was left by them: the MFMA-bound layers run below the 2.4 GHz maximum under the
 * power limit.  out: 16 bytes of device memory, 8-byte aligned. */
void pulp_nn_hip_clock_probe(long long *out);

/* Status of the most recent failing layer call on this thread since the last
 * pulp_nn_hip_clear_error(), or PULP_NN_HIP_OK.  A layer call that fails
 * validation queues no work. */
int pulp_nn_hip_last_error(void);
const char *pulp_nn_hip_last_error_string(void);
void pulp_nn_hip_clear_error(void);

/* 32 or 64: the width of k / lambda this build of the library expects. */
int pulp_nn_hip_bn_bits(void);

/* Layout glue between a conv / pointwise output (HWC) and a depthwise input
 * (CHW), which the reference leaves to the application: writes, per image,
 * ch planes of (pad_top + dim_y + pad_bottom) x dim_x bytes, the pad rows
 * zero.  pad_top = pad_bottom = 1 gives the row-padded plane that
 * pulp_nn_depthwise_3x3_s1 expects. */
void pulp_nn_hip_hwc_to_chw(const unsigned char *in_hwc, unsigned char *out_chw,
                            unsigned dim_x, unsigned dim_y, unsigned ch,
                            unsigned pad_top, unsigned pad_bottom);

/* The glue above fused into the layer that follows it: a 3x3 depthwise convolution with
 * padding 1 on all sides and stride 1 or 2 that reads its input as HWC (the output of the
 * previous conv / pointwise layer) and writes HWC.  Arithmetic and the remaining arguments are
 * those of pulp_nn_depthwise_generic (k, lambda: int32_t or int64_t arrays as the build
 * expects; out_shift is taken as int8_t).  Available where the library keeps the rows of a
 * plane in registers: 8x8 and 4x4 (stride 1) images with a multiple of 64 channels, and
 * images 16, 32 or 64 pixels wide with a multiple of 4 channels and batch x channels a
 * multiple of 64.  Any other geometry sets PULP_NN_HIP_ERR_UNSUPPORTED and queues nothing:
 * call pulp_nn_hip_hwc_to_chw and pulp_nn_depthwise_generic instead. */
void pulp_nn_hip_depthwise_hwc(const unsigned char *Im_in, const signed char *bias, unsigned char *Im_out,
                               const signed char *wt, void *k, void *lambda, unsigned short out_mult,
                               unsigned short out_shift, unsigned short dim_im_in_x, unsigned short dim_im_in_y,
                               unsigned short ch, unsigned short dim_im_out_x, unsigned short dim_im_out_y,
                               unsigned short stride, signed char flag_relu, signed char flag_batch_norm);

/* A depthwise 3x3 layer (padding 1 on every side, stride 1 or 2, HWC input as
 * pulp_nn_hip_depthwise_hwc takes it) and the pointwise layer that follows it, in one launch:
 * no counterpart in the reference, where the depthwise result goes to memory in HWC
 * (32bit/src/pulp_nn_depthwise_generic.c:179) and the pointwise layer reads it back
 * (pulp_nn_pointwise_HoWo_parallel.c:103).  The result is bit for bit that of
 * pulp_nn_hip_depthwise_hwc followed by pulp_nn_pointwise_HoWo_parallel with the same
 * parameters (dw_*: the depthwise layer's; pw_*: the pointwise layer's, pw_weight[ch_out][ch]);
 * the intermediate tensor is never written.  k / lambda arrays are int32_t or int64_t as the
 * build expects.  Supported: dim_im_in_x in {64, 32, 16, 8} (and 4 with stride 1), ch in
 * {16, 32} or a multiple of 64 up to 1024, ch_out a multiple of 16 and at most 1024 per
 * workgroup (small layers are split over several workgroups by output channels, so more can
 * pass; a large batch with ch_out > 1024 cannot), output rows a multiple of
 * the rows a wave takes at once (2 to 8, times 64 / ch for ch < 64), 16-byte aligned pointwise
 * weights and output.  Anything else sets PULP_NN_HIP_ERR_UNSUPPORTED and queues nothing:
 * make the two calls instead. */
void pulp_nn_hip_dw_pw_hwc(const unsigned char *Im_in, unsigned char *Im_out, unsigned short dim_im_in_x,
                           unsigned short dim_im_in_y, unsigned short ch, unsigned short dim_im_out_x,
                           unsigned short dim_im_out_y, unsigned short ch_out, unsigned short stride,
                           const signed char *dw_wt, const signed char *dw_bias, void *dw_k, void *dw_lambda,
                           unsigned short dw_out_mult, unsigned short dw_out_shift, signed char dw_flag_relu,
                           signed char dw_flag_batch_norm, const signed char *pw_weight, const signed char *pw_bias,
                           void *pw_k, void *pw_lambda, unsigned short pw_out_mult, unsigned short pw_out_shift,
                           signed char pw_flag_relu, signed char pw_flag_batch_norm);

/* The parameters of one such block, as pulp_nn_hip_dw_pw_hwc takes them. */
typedef struct pulp_nn_hip_block {
  const signed char *dw_wt, *dw_bias;
  void *dw_k, *dw_lambda;
  unsigned short dw_out_mult, dw_out_shift;
  signed char dw_flag_relu, dw_flag_batch_norm;
  const signed char *pw_weight, *pw_bias;
  void *pw_k, *pw_lambda;
  unsigned short pw_out_mult, pw_out_shift;
  signed char pw_flag_relu, pw_flag_batch_norm;
} pulp_nn_hip_block;

/* n_blocks (1 to 8) such blocks of the same shape one after the other in one launch: stride 1, ch
 * channels in and out of every layer, dim_im_x x dim_im_y pixels throughout (the run of identical
 * blocks in the middle of a MobileNet).  No counterpart in the reference, which makes 2 x n_blocks
 * calls with every intermediate tensor in memory.  Here a workgroup keeps its images' activations
 * in LDS from block to block; only the last block's output is written.  blocks is a host array.
 * The result is bit for bit that of n_blocks calls of pulp_nn_hip_dw_pw_hwc.  Supported: what
 * pulp_nn_hip_dw_pw_hwc supports at stride 1 with ch_out == ch, images small enough for a
 * workgroup to hold whole ones (dim_im_x x dim_im_y x ch x 2 bytes and the constants within 64 KB
 * of LDS: 8 x 8 x 256, 16 x 16 x 64, 4 x 4 x 512 ...), and a batch that is a multiple of the
 * images a workgroup takes.  Anything else sets PULP_NN_HIP_ERR_UNSUPPORTED and queues nothing:
 * call pulp_nn_hip_dw_pw_hwc per block instead. */
void pulp_nn_hip_dw_pw_chain_hwc(const unsigned char *Im_in, unsigned char *Im_out, unsigned short dim_im_x,
                                 unsigned short dim_im_y, unsigned short ch, unsigned n_blocks,
                                 const pulp_nn_hip_block *blocks);

/* ---- calibration of out_shift -------------------------------------------------------
 * A network that requantises with batch-norm + ReLU chooses, per layer,
 * out_shift = floor(log2(max |acc * k[c]|)) - 7, the maximum taken over the batch, all
 * output pixels and all output channels; acc is the layer's accumulator including bias
 * (what pulp_nn_matmul / pulp_nn_depthwise_generic hand to pulp_nn_bn_quant_u8).  The
 * reference leaves this to offline tooling; the calls below compute it on the GPU from the
 * layer's own device tensors, for pulp_nn_hip_set_batch() images.
 *
 * result points to two 64-bit words in DEVICE memory, written on the stream:
 * result[0] = max |acc * k[c]| (64-bit wrapping product, as the 64-bit tree forms it),
 * result[1] = max(floor(log2(result[0])) - 7, 0), and 0 for a layer whose maximum is 0.
 * The 32-bit build reports the same unwrapped 64-bit magnitude, although its layers form
 * acc * k in int32 (32bit/src/pulp_nn_utils.c:35-45): result[0] >= 2^31 means that the
 * layer's product wraps on this batch and result[1] does not describe it; callers check
 * result[0] < 2^31 there.
 * k is an int32_t or int64_t array as the build expects.  The geometry arguments have the
 * meaning they have in pulp_nn_conv_Ho_parallel (a pointwise layer is a 1x1 kernel with
 * stride 1 and no padding; a linear layer is a pointwise layer on a 1x1 image) and in
 * pulp_nn_depthwise_generic.
 *
 * workspace: device memory for the partial maxima, 8-byte aligned, at least
 * pulp_nn_hip_calib_workspace_bytes(batch * dim_out_x * dim_out_y * ch_out) bytes (one
 * 8-byte slot per 65536 outputs); its previous contents do not matter.  Calls that share a
 * workspace must not overlap in time. */
unsigned long long pulp_nn_hip_calib_workspace_bytes(unsigned long long n_outputs);

void pulp_nn_hip_calib_conv(const unsigned char *pInBuffer, const signed char *bias, const signed char *pWeight,
                            const void *k, unsigned short dim_in_x, unsigned short dim_in_y, unsigned short ch_in,
                            unsigned short dim_out_x, unsigned short dim_out_y, unsigned short ch_out,
                            unsigned short dim_kernel_x, unsigned short dim_kernel_y, unsigned short padding_y_top,
                            unsigned short padding_x_left, unsigned short stride_x, unsigned short stride_y,
                            void *workspace, unsigned long long workspace_bytes, unsigned long long *result);

/* Depthwise layer (one [ky][kx] filter per channel).  input_is_hwc = 0: CHW input as
 * pulp_nn_depthwise_generic takes it; 1: HWC input as pulp_nn_hip_depthwise_hwc takes it. */
void pulp_nn_hip_calib_depthwise(const unsigned char *Im_in, const signed char *bias, const signed char *wt,
                                 const void *k, unsigned short dim_im_in_x, unsigned short dim_im_in_y,
                                 unsigned short ch, unsigned short dim_im_out_x, unsigned short dim_im_out_y,
                                 unsigned short dim_kernel_x, unsigned short dim_kernel_y, unsigned short padding_y_top,
                                 unsigned short padding_x_left, unsigned short stride_x, unsigned short stride_y,
                                 int input_is_hwc, void *workspace, unsigned long long workspace_bytes,
                                 unsigned long long *result);

/* pulp_nn_hip_calib_conv for callers that cannot allocate device memory or carry a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): no counterpart in the reference.  Same arguments and same result as
 * pulp_nn_hip_calib_conv without the workspace: the partial maxima go to a fixed array of
 * 8192 slots (64 KiB) that the library holds in the device memory of every GPU it runs on
 * until the process ends.  The call allocates and frees nothing.  A layer with more than
 * 8192 * 65536 outputs (batch * dim_out_x * dim_out_y * ch_out) is rejected with
 * PULP_NN_HIP_ERR_ARGUMENT.  All calls on one GPU share that array: calls that overlap in
 * time on one GPU (different streams or host threads) race and must be serialised by the
 * caller. */
void pulp_nn_hip_calib_conv_static(const unsigned char *pInBuffer, const signed char *bias, const signed char *pWeight,
                                   const void *k, unsigned short dim_in_x, unsigned short dim_in_y,
                                   unsigned short ch_in, unsigned short dim_out_x, unsigned short dim_out_y,
                                   unsigned short ch_out, unsigned short dim_kernel_x, unsigned short dim_kernel_y,
                                   unsigned short padding_y_top, unsigned short padding_x_left,
                                   unsigned short stride_x, unsigned short stride_y, unsigned long long *result);

#ifdef __cplusplus
}
#endif
#endif
