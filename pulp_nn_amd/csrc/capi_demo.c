/* A plain C99 caller of the library, the way a PULP-NN application calls its kernels
 * (32bit/include/pulp_nn_kernels.h:155-181 pulp_nn_pointwise_HoWo_parallel, :271-299 pulp_nn_depthwise_generic):
 * device buffers from the HIP runtime instead of cluster L1, one added call for the batch, NULL for the scratch
 * arguments.  It runs a pointwise layer, then a 3x3 depthwise layer (after the HWC -> CHW glue) on its output,
 * and writes both results to a file for the test that drives it (tests/test_gpu_c_caller.py).
 *
 * Input file: int32 header {B, H, W, Ci, Co, pw_mult, pw_shift, dw_shift}, then x[B*H*W*Ci] (uint8),
 * w[Co*Ci] (int8), bias[Co] (int8), dw_w[Co*9] (int8), dw_k[Co] (int32), dw_lambda[Co] (int32).
 * Output file: pointwise out[B*H*W*Co] (uint8, HWC), then depthwise out[B*H*W*Co] (uint8, HWC).
 *
 * Build: gcc -std=c99 -D__HIP_PLATFORM_AMD__ -I include -I /opt/rocm/include capi_demo.c -L lib -lpulpnn_hip32 -lamdhip64
 * (python -m pulp_nn_amd.build does it). */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "32bit/pulp_nn_kernels.h"

#define CHECK(x)                                                                  \
  do {                                                                            \
    hipError_t e_ = (x);                                                          \
    if (e_ != hipSuccess) {                                                       \
      fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));              \
      return 2;                                                                   \
    }                                                                             \
  } while (0)

static void *to_device(const void *host, size_t n)
{
  void *d = NULL;
  if (hipMalloc(&d, n ? n : 1) != hipSuccess) return NULL;
  if (host && n && hipMemcpy(d, host, n, hipMemcpyHostToDevice) != hipSuccess) return NULL;
  return d;
}

int main(int argc, char **argv)
{
  if (argc != 3) {
    fprintf(stderr, "usage: %s input.bin output.bin\n", argv[0]);
    return 1;
  }
  FILE *f = fopen(argv[1], "rb");
  if (!f) return 1;
  int32_t h[8];
  if (fread(h, 4, 8, f) != 8) return 1;
  const int B = h[0], H = h[1], W = h[2], Ci = h[3], Co = h[4], pw_mult = h[5], pw_shift = h[6], dw_shift = h[7];
  const size_t nx = (size_t)B * H * W * Ci, ny = (size_t)B * H * W * Co;
  uint8_t *x = malloc(nx), *y = malloc(2 * ny);
  int8_t *w = malloc((size_t)Co * Ci), *bias = malloc(Co), *dww = malloc((size_t)Co * 9);
  int32_t *k = malloc(4 * (size_t)Co), *lam = malloc(4 * (size_t)Co);
  if (!x || !y || !w || !bias || !dww || !k || !lam) return 1;
  if (fread(x, 1, nx, f) != nx || fread(w, 1, (size_t)Co * Ci, f) != (size_t)Co * Ci || fread(bias, 1, Co, f) != (size_t)Co ||
      fread(dww, 1, (size_t)Co * 9, f) != (size_t)Co * 9 || fread(k, 4, Co, f) != (size_t)Co || fread(lam, 4, Co, f) != (size_t)Co)
    return 1;
  fclose(f);

  uint8_t *d_x = to_device(x, nx), *d_pw = to_device(NULL, ny), *d_chw = to_device(NULL, ny), *d_dw = to_device(NULL, ny);
  int8_t *d_w = to_device(w, (size_t)Co * Ci), *d_bias = to_device(bias, Co), *d_dww = to_device(dww, (size_t)Co * 9);
  int32_t *d_k = to_device(k, 4 * (size_t)Co), *d_lam = to_device(lam, 4 * (size_t)Co);
  if (!d_x || !d_pw || !d_chw || !d_dw || !d_w || !d_bias || !d_dww || !d_k || !d_lam) return 2;

  pulp_nn_hip_set_batch((unsigned)B); /* images back to back, as the reference's caller would loop over them */
  /* 1x1 convolution, scalar-multiplier requantisation + ReLU (flag_relu = 1, flag_batch_norm = 0) */
  pulp_nn_pointwise_HoWo_parallel(d_x, NULL, d_bias, d_pw, d_w, NULL, NULL, (uint16_t)pw_mult, (uint16_t)pw_shift,
                                  (uint16_t)W, (uint16_t)H, (uint16_t)Ci, (uint16_t)W, (uint16_t)H, (uint16_t)Co,
                                  1, 1, 0, 0, 0, 0, 1, 1, 1, 0);
  /* the reference's depthwise kernels read CHW: the layout change its applications do between the two layers */
  pulp_nn_hip_hwc_to_chw(d_pw, d_chw, (uint16_t)W, (uint16_t)H, (uint16_t)Co, 0, 0);
  /* 3x3 depthwise, padding 1, stride 1, batch-norm requantisation + ReLU */
  pulp_nn_depthwise_generic(d_chw, NULL, NULL, d_dw, d_dww, NULL, d_k, d_lam, 0, (uint16_t)dw_shift, (uint16_t)W, (uint16_t)H,
                            (uint16_t)Co, (uint16_t)W, (uint16_t)H, (uint16_t)Co, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1);
  if (pulp_nn_hip_last_error()) {
    fprintf(stderr, "%s\n", pulp_nn_hip_last_error_string());
    return 3;
  }
  if (pulp_nn_hip_sync()) return 3;
  CHECK(hipMemcpy(y, d_pw, ny, hipMemcpyDeviceToHost));
  CHECK(hipMemcpy(y + ny, d_dw, ny, hipMemcpyDeviceToHost));
  f = fopen(argv[2], "wb");
  if (!f || fwrite(y, 1, 2 * ny, f) != 2 * ny) return 1;
  fclose(f);
  return 0;
}
