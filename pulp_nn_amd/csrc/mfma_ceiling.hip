// Measures what the int8 matrix cores of this GPU sustain, as a yardstick for the convolution kernels:
//
//   1. v_mfma_i32_16x16x64_i8 from registers only (no memory traffic at all), with constant operands and
//      with random bytes, at 1, 2 and 4 waves per SIMD.  Reports op/s, the shader clock during the loop
//      (cycle counter against the 100 MHz wall clock) and cycles per MFMA per SIMD.  What it shows on
//      MI355X: one wave per SIMD cannot issue back-to-back MFMAs faster than one per ~26 cycles (two
//      waves reach the pipe's 16); with random operand bytes the clock drops from 2.4 GHz to about
//      2.0-2.1 GHz at full rate (the power limit), so about 4.0 POP/s is the most any int8 kernel can
//      sustain on random data.
//   2. The operand feed of a 256 x 256 tile kernel without any global memory traffic: eight waves of
//      128 x 64, per 64-byte K slice twelve ds_read_b128 fragment reads, the ^ 0x80 on the activation
//      fragments and 32 MFMAs per wave, with and without a workgroup barrier per slice and with the
//      fragment reads issued one slice ahead.  That is the main loop of igemm_dma_kernel with its
//      global loads taken out: the rate it reaches bounds what that kernel structure can reach.
//   3. The issue rate of the vector ALU for the instructions the depthwise kernels are made of (v_dot4,
//      24-bit multiply-add, byte permute / align, DPP move, xor), at 1, 2 and 4 waves per SIMD, from the
//      duration of a kernel of independent instruction chains: cycles per wave64 instruction per SIMD.
//      With a kernel's SQ_INSTS_VALU count this gives the time its vector work alone needs.
//
// Build: hipcc --offload-arch=gfx950 -O3 -std=c++17 mfma_ceiling.hip -o ../lib/mfma_ceiling
// (python -m pulp_nn_amd.build does it).  Run without arguments.
#include <hip/hip_runtime.h>
#include <stdio.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
#define CK(x)                                                              \
  do {                                                                     \
    hipError_t e_ = (x);                                                   \
    if (e_ != hipSuccess) {                                                \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      return 1;                                                            \
    }                                                                      \
  } while (0)

__device__ unsigned hash32(unsigned x)
{
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

// ---- 1. registers only: acc[i][j] += a[i] * b[j], NA x NB accumulators per wave, W waves per workgroup,
//         one workgroup per compute unit (the 100 KB of LDS requested keep a second one out) -------------
template <int NA, int NB, int RND, int W>
__global__ __launch_bounds__(64 * W) void reg_kernel(int *out, long long *clk, int iters)
{
  extern __shared__ int lds[];
  v4i a[NA], b[NB];
  for (int q = 0; q < NA; q++) {
    const unsigned s = threadIdx.x * 131 + q * 7919 + blockIdx.x;
    a[q] = RND ? (v4i){(int)hash32(s), (int)hash32(s + 1), (int)hash32(s + 2), (int)hash32(s + 3)} : (v4i){(int)threadIdx.x & 3, 1, 2, 3};
  }
  for (int q = 0; q < NB; q++) {
    const unsigned s = threadIdx.x * 137 + q * 7907 + blockIdx.x + 99;
    b[q] = RND ? (v4i){(int)hash32(s), (int)hash32(s + 1), (int)hash32(s + 2), (int)hash32(s + 3)} : (v4i){5, (int)threadIdx.x & 3, 7, 8};
  }
  v4i acc[NA][NB];
  for (int i = 0; i < NA; i++)
    for (int j = 0; j < NB; j++) acc[i][j] = (v4i){0, 0, 0, 0};
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < NA; i++)
#pragma unroll
      for (int j = 0; j < NB; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  int s = 0;
  for (int i = 0; i < NA; i++)
    for (int j = 0; j < NB; j++) s += acc[i][j].x + acc[i][j].y + acc[i][j].z + acc[i][j].w;
  out[blockIdx.x * blockDim.x + threadIdx.x] = s + lds[threadIdx.x & 1];
  if (threadIdx.x == 0) {
    clk[2 * blockIdx.x] = c1 - c0;
    clk[2 * blockIdx.x + 1] = w1 - w0;
  }
}


// the same with v_mfma_i32_32x32x32_i8 (16 accumulator registers per MFMA, 65536 op, 32 cycles per SIMD at peak)
template <int NA, int NB, int RND, int W>
__global__ __launch_bounds__(64 * W) void reg32_kernel(int *out, long long *clk, int iters)
{
  extern __shared__ int lds[];
  v4i a[NA], b[NB];
  for (int q = 0; q < NA; q++) {
    const unsigned s = threadIdx.x * 131 + q * 7919 + blockIdx.x;
    a[q] = RND ? (v4i){(int)hash32(s), (int)hash32(s + 1), (int)hash32(s + 2), (int)hash32(s + 3)} : (v4i){(int)threadIdx.x & 3, 1, 2, 3};
  }
  for (int q = 0; q < NB; q++) {
    const unsigned s = threadIdx.x * 137 + q * 7907 + blockIdx.x + 99;
    b[q] = RND ? (v4i){(int)hash32(s), (int)hash32(s + 1), (int)hash32(s + 2), (int)hash32(s + 3)} : (v4i){5, (int)threadIdx.x & 3, 7, 8};
  }
  v16i acc[NA][NB];
  for (int i = 0; i < NA; i++)
    for (int j = 0; j < NB; j++)
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < NA; i++)
#pragma unroll
      for (int j = 0; j < NB; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  int s = 0;
  for (int i = 0; i < NA; i++)
    for (int j = 0; j < NB; j++)
      for (int r = 0; r < 16; r++) s += acc[i][j][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s + lds[threadIdx.x & 1];
  if (threadIdx.x == 0) {
    clk[2 * blockIdx.x] = c1 - c0;
    clk[2 * blockIdx.x + 1] = w1 - w0;
  }
}

// ---- 2. operand feed from LDS: eight waves, wave tile 128 px x 64 ch ---------------------------------
// PIPE: the fragments of the next slice are requested before this slice's MFMAs; BAR: s_barrier per slice
template <int PIPE, int BAR>
__global__ __launch_bounds__(512) void feed_kernel(int *out, long long *clk, int iters)
{
  extern __shared__ __attribute__((aligned(16))) unsigned char feed_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l16 = lane & 15, lgrp = lane >> 4;
  for (int i = tid; i < 65536 / 4; i += 512) ((unsigned *)feed_lds)[i] = hash32(i + blockIdx.x * 77);
  __syncthreads();
  const int swz = (lgrp ^ ((l16 >> 1) & 3)) << 4;
  const unsigned char *a_lane = feed_lds + ((wave & 1) * 128 + l16) * 64 + swz;
  const unsigned char *w_lane = feed_lds + 32768 + ((wave >> 1) * 64 + l16) * 64 + swz;
  v4i acc[4][8];
  for (int i = 0; i < 4; i++)
    for (int j = 0; j < 8; j++) acc[i][j] = (v4i){0, 0, 0, 0};
  struct Frags {
    v4i wf[4], af[8];
  };
  // (the slot offset is read through a volatile so that the compiler cannot hoist the reads out of the loop)
  volatile int slot_mask = 1;
  auto read = [&](Frags &F, int j) {
    const int slot = (j & slot_mask) * 16384;
#pragma unroll
    for (int t = 0; t < 4; t++) F.wf[t] = *(const v4i *)(w_lane + slot + t * 1024);
#pragma unroll
    for (int s = 0; s < 8; s++) F.af[s] = *(const v4i *)(a_lane + slot + s * 1024);
  };
  auto multiply = [&](Frags &F) {
#pragma unroll
    for (int s = 0; s < 8; s++) {
      const v4i a = F.af[s] ^ (int)0x80808080;
#pragma unroll
      for (int t = 0; t < 4; t++) acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(F.wf[t], a, acc[t][s], 0, 0, 0);
    }
  };
  Frags F0, F1;
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  if (PIPE == 0) {
    for (int it = 0; it < iters; it++) {
      if (BAR) __builtin_amdgcn_s_barrier();
      read(F0, it);
      multiply(F0);
    }
  } else {
    read(F0, 0);
    for (int it = 0; it < iters; it += 2) {
      if (BAR) __builtin_amdgcn_s_barrier();
      read(F1, it + 1);
      multiply(F0);
      if (BAR) __builtin_amdgcn_s_barrier();
      read(F0, it + 2);
      multiply(F1);
    }
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  int s = 0;
  for (int i = 0; i < 4; i++)
    for (int j = 0; j < 8; j++) s += acc[i][j].x + acc[i][j].y + acc[i][j].z + acc[i][j].w;
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    clk[2 * blockIdx.x] = c1 - c0;
    clk[2 * blockIdx.x + 1] = w1 - w0;
  }
}


// the same wave tile on v_mfma_i32_32x32x32_i8: a fragment is 32 rows x 32 bytes of K (lane l: row l%32,
// 16-byte chunk l/32 of the K step), per 64-byte K slice again twelve ds_read_b128, 32 xor, and 16 MFMAs
template <int PIPE, int BAR>
__global__ __launch_bounds__(512) void feed32_kernel(int *out, long long *clk, int iters)
{
  extern __shared__ __attribute__((aligned(16))) unsigned char feed_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, lh = lane >> 5;
  for (int i = tid; i < 65536 / 4; i += 512) ((unsigned *)feed_lds)[i] = hash32(i + blockIdx.x * 77);
  __syncthreads();
  // K step ks of row r: chunk 2*ks + lh in slot chunk ^ ((r/2)%4)
  const int sw = (l32 >> 1) & 3;
  const int o0 = ((0 + lh) ^ sw) << 4, o1 = ((2 + lh) ^ sw) << 4;
  const unsigned char *a_lane = feed_lds + ((wave & 1) * 128 + l32) * 64;
  const unsigned char *w_lane = feed_lds + 32768 + ((wave >> 1) * 64 + l32) * 64;
  v16i acc[2][4];
  for (int i = 0; i < 2; i++)
    for (int j = 0; j < 4; j++)
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
  struct Frags {
    v4i wf[2][2], af[4][2];
  };
  volatile int slot_mask = 1;
  auto read = [&](Frags &F, int j) {
    const int slot = (j & slot_mask) * 16384;
#pragma unroll
    for (int t = 0; t < 2; t++) {
      F.wf[t][0] = *(const v4i *)(w_lane + slot + t * 2048 + o0);
      F.wf[t][1] = *(const v4i *)(w_lane + slot + t * 2048 + o1);
    }
#pragma unroll
    for (int s = 0; s < 4; s++) {
      F.af[s][0] = *(const v4i *)(a_lane + slot + s * 2048 + o0);
      F.af[s][1] = *(const v4i *)(a_lane + slot + s * 2048 + o1);
    }
  };
  auto multiply = [&](Frags &F) {
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
      for (int s = 0; s < 4; s++) {
        const v4i a = F.af[s][ks] ^ (int)0x80808080;
#pragma unroll
        for (int t = 0; t < 2; t++) acc[t][s] = __builtin_amdgcn_mfma_i32_32x32x32_i8(F.wf[t][ks], a, acc[t][s], 0, 0, 0);
      }
  };
  Frags F0, F1;
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  if (PIPE == 0) {
    for (int it = 0; it < iters; it++) {
      if (BAR) __builtin_amdgcn_s_barrier();
      read(F0, it);
      multiply(F0);
    }
  } else {
    read(F0, 0);
    for (int it = 0; it < iters; it += 2) {
      if (BAR) __builtin_amdgcn_s_barrier();
      read(F1, it + 1);
      multiply(F0);
      if (BAR) __builtin_amdgcn_s_barrier();
      read(F0, it + 2);
      multiply(F1);
    }
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  int s = 0;
  for (int i = 0; i < 2; i++)
    for (int j = 0; j < 4; j++)
      for (int r = 0; r < 16; r++) s += acc[i][j][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    clk[2 * blockIdx.x] = c1 - c0;
    clk[2 * blockIdx.x + 1] = w1 - w0;
  }
}

// LDS read bandwidth: W waves per SIMD reading conflict-free 16-byte fragments back to back
__global__ __launch_bounds__(1024) void ldsbw_kernel(int *out, long long *clk, int iters)
{
  extern __shared__ __attribute__((aligned(16))) unsigned char feed_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l16 = lane & 15, lgrp = lane >> 4;
  for (int i = tid; i < 65536 / 4; i += blockDim.x) ((unsigned *)feed_lds)[i] = hash32(i);
  __syncthreads();
  const unsigned char *p = feed_lds + (((wave & 7) * 64 + l16) * 64) + ((lgrp ^ ((l16 >> 1) & 3)) << 4);
  v4i acc = {0, 0, 0, 0};
  volatile int slot_mask = 1;
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
    const int slot = (it & slot_mask) * 32768;
    v4i v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) v[u] = *(const v4i *)(p + slot + (u & 3) * 1024);
#pragma unroll
    for (int u = 0; u < 8; u++) acc ^= v[u];
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  out[blockIdx.x * blockDim.x + threadIdx.x] = acc.x + acc.y + acc.z + acc.w;
  if (threadIdx.x == 0) {
    clk[2 * blockIdx.x] = c1 - c0;
    clk[2 * blockIdx.x + 1] = w1 - w0;
  }
}

// ---- 3. vector ALU issue rate ---------------------------------------------------------------------------
template <int OP>
__global__ __launch_bounds__(1024) void valu_kernel(int *out, long long *clk, int iters)
{
  int a[8], b = threadIdx.x * 77 + 1, c = threadIdx.x ^ 0x1234567;
  for (int i = 0; i < 8; i++) a[i] = threadIdx.x + i;
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
      for (int i = 0; i < 8; i++) {
        if (OP == 0) asm volatile("v_dot4c_i32_i8 %0, %1, %2" : "+v"(a[i]) : "v"(b), "v"(c));
        if (OP == 1) asm volatile("v_dot4_i32_i8 %0, %1, %2, %0" : "+v"(a[i]) : "v"(b), "v"(c));
        if (OP == 2) asm volatile("v_mad_i32_i24 %0, %1, %2, %0" : "+v"(a[i]) : "v"(b), "v"(c));
        if (OP == 3) asm volatile("v_perm_b32 %0, %1, %2, %0" : "+v"(a[i]) : "v"(b), "v"(c));
        if (OP == 4) asm volatile("v_alignbyte_b32 %0, %1, %0, 3" : "+v"(a[i]) : "v"(b));
        if (OP == 5) asm volatile("v_mov_b32_dpp %0, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "+v"(a[i]) : "v"(b));
        if (OP == 6) asm volatile("v_xor_b32 %0, %1, %0" : "+v"(a[i]) : "v"(b));
      }
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  int s = 0;
  for (int i = 0; i < 8; i++) s += a[i];
  out[blockIdx.x * 1024 + threadIdx.x] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    clk[0] = c1 - c0;
    clk[1] = w1 - w0;
  }
}

static int g_cus = 256;

template <int OP>
int run_valu(const char *name, int *out, long long *clk)
{
  const int iters = 20000;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  printf("%-18s", name);
  for (int w = 1; w <= 4; w *= 2) {
    hipLaunchKernelGGL(valu_kernel<OP>, dim3(g_cus), dim3(256 * w), 0, 0, out, clk, iters);
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(valu_kernel<OP>, dim3(g_cus), dim3(256 * w), 0, 0, out, clk, iters);
    CK(hipEventRecord(e1, 0));
    CK(hipDeviceSynchronize());
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    long long h[2];
    CK(hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost));
    const double mhz = (double)h[0] / (h[1] / 100.0);
    printf("  %d waves/SIMD: %.2f cycles/instr/SIMD (%4.0f MHz)", w, ms * 1e-3 * mhz * 1e6 / (iters * 32.0 * w), mhz);
  }
  printf("\n");
  fflush(stdout);
  return 0;
}

template <typename K>
int run(const char *name, K kern, int waves, long long mfma_per_wave_iter, int iters, int *out, long long *clk, int op_per_mfma = 32768)
{
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  const int reps = 5;
  CK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024));
  hipLaunchKernelGGL(kern, dim3(g_cus), dim3(64 * waves), 100 * 1024, 0, out, clk, iters);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0, 0));
  for (int r = 0; r < reps; r++) hipLaunchKernelGGL(kern, dim3(g_cus), dim3(64 * waves), 100 * 1024, 0, out, clk, iters);
  CK(hipEventRecord(e1, 0));
  CK(hipDeviceSynchronize());
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  long long h[2];
  CK(hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost));
  const double mfmas = (double)reps * g_cus * waves * iters * mfma_per_wave_iter;
  const double mhz = (double)h[0] / (h[1] / 100.0);
  const double pops = mfmas * op_per_mfma / (ms * 1e-3) / 1e15;
  printf("%-58s %d waves/SIMD  %6.3f POP/s  %4.0f MHz  %5.1f cycles/MFMA/SIMD\n", name, waves / 4, pops, mhz,
         (ms * 1e-3) * mhz * 1e6 / (mfmas / (g_cus * 4.0)));
  fflush(stdout);
  return 0;
}

int main()
{
  int dev = 0;
  hipDeviceProp_t prop;
  CK(hipGetDevice(&dev));
  CK(hipGetDeviceProperties(&prop, dev));
  g_cus = prop.multiProcessorCount;
  printf("%s (%s), %d compute units; published dense int8 peak 5.0 POP/s = 16 cycles per 16x16x64 MFMA per SIMD at 2.4 GHz\n",
         prop.name[0] ? prop.name : "GPU", prop.gcnArchName, g_cus);
  int *out;
  long long *clk;
  CK(hipMalloc(&out, 4096 * 1024 * 4));
  CK(hipMalloc(&clk, 4096 * 16));
  printf("-- registers only (no LDS, no memory) --\n");
  run("constant operands, 16 accumulators", reg_kernel<4, 4, 0, 16>, 16, 16, 2500, out, clk);
  run("constant operands, 32 accumulators", reg_kernel<4, 8, 0, 8>, 8, 32, 1250, out, clk);
  run("constant operands, 32 accumulators", reg_kernel<4, 8, 0, 4>, 4, 32, 1250, out, clk);
  run("random bytes, 16 accumulators", reg_kernel<4, 4, 1, 16>, 16, 16, 2500, out, clk);
  run("random bytes, 32 accumulators", reg_kernel<4, 8, 1, 8>, 8, 32, 1250, out, clk);
  run("random bytes, 32 accumulators", reg_kernel<4, 8, 1, 4>, 4, 32, 1250, out, clk);
  printf("-- registers only, v_mfma_i32_32x32x32_i8 (cycles per MFMA: 32 at peak) --\n");
  run("32x32x32, constant operands, 8 accumulators of 16", reg32_kernel<2, 4, 0, 8>, 8, 8, 2500, out, clk, 65536);
  run("32x32x32, constant operands, 8 accumulators of 16", reg32_kernel<2, 4, 0, 4>, 4, 8, 2500, out, clk, 65536);
  run("32x32x32, random bytes, 8 accumulators of 16", reg32_kernel<2, 4, 1, 8>, 8, 8, 2500, out, clk, 65536);
  run("32x32x32, random bytes, 8 accumulators of 16", reg32_kernel<2, 4, 1, 4>, 4, 8, 2500, out, clk, 65536);
  printf("-- operands from LDS: 12 ds_read_b128 + 32 xor + 32 MFMA per wave and K slice, random bytes --\n");
  run("reads, then MFMAs; no barrier", feed_kernel<0, 0>, 8, 32, 2000, out, clk);
  run("reads, then MFMAs; barrier per slice", feed_kernel<0, 1>, 8, 32, 2000, out, clk);
  run("reads one slice ahead; no barrier", feed_kernel<1, 0>, 8, 32, 2000, out, clk);
  run("reads one slice ahead; barrier per slice", feed_kernel<1, 1>, 8, 32, 2000, out, clk);
  printf("-- the same wave tile on v_mfma_i32_32x32x32_i8: 12 ds_read_b128 + 32 xor + 16 MFMA per wave and K slice --\n");
  run("32x32x32: reads, then MFMAs; no barrier", feed32_kernel<0, 0>, 8, 16, 2000, out, clk, 65536);
  run("32x32x32: reads, then MFMAs; barrier per slice", feed32_kernel<0, 1>, 8, 16, 2000, out, clk, 65536);
  run("32x32x32: reads one slice ahead; no barrier", feed32_kernel<1, 0>, 8, 16, 2000, out, clk, 65536);
  run("32x32x32: reads one slice ahead; barrier per slice", feed32_kernel<1, 1>, 8, 16, 2000, out, clk, 65536);
  printf("-- LDS read rate: conflict-free ds_read_b128 back to back, one workgroup per compute unit --\n");
  for (int w = 4; w <= 16; w *= 2) {
    const int iters = 4000;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    CK(hipFuncSetAttribute((const void *)ldsbw_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024));
    hipLaunchKernelGGL(ldsbw_kernel, dim3(g_cus), dim3(64 * w), 100 * 1024, 0, out, clk, iters);
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(ldsbw_kernel, dim3(g_cus), dim3(64 * w), 100 * 1024, 0, out, clk, iters);
    CK(hipEventRecord(e1, 0));
    CK(hipDeviceSynchronize());
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    long long h[2];
    CK(hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost));
    const double mhz = (double)h[0] / (h[1] / 100.0);
    printf("ds_read_b128, %d waves/SIMD: %.1f bytes per cycle per compute unit (%4.0f MHz)\n", w / 4,
           (double)w * iters * 8 * 1024 / (ms * 1e-3 * mhz * 1e6), mhz);
  }
  printf("-- vector ALU: cycles per wave64 instruction per SIMD (one workgroup per compute unit, independent chains) --\n");
  run_valu<0>("v_dot4c_i32_i8", out, clk);
  run_valu<1>("v_dot4_i32_i8", out, clk);
  run_valu<2>("v_mad_i32_i24", out, clk);
  run_valu<3>("v_perm_b32", out, clk);
  run_valu<4>("v_alignbyte_b32", out, clk);
  run_valu<5>("v_mov_b32_dpp", out, clk);
  run_valu<6>("v_xor_b32", out, clk);
  return 0;
}
