// Memory yardstick for the HBM-bound layers: what plain streaming kernels reach on buffers of the same size.
//
// The roofline of the depthwise, pooling and pointwise layers is priced against the published 8 TB/s.  This tool
// measures how much of that a kernel with no arithmetic and the friendliest access pattern there is gets on the
// same machine: every workgroup copies (reads, writes) whole 4 KB blocks with 16-byte accesses per lane.  Rows:
//   copy    in -> out, default cache policy and nontemporal loads and stores
//   read    in -> nothing (a checksum that is never stored)
//   write   nothing -> out
//   memcpy  hipMemcpyAsync device to device, what a framework's copy_ does
// for the byte counts of three layers: the stride-1 and stride-2 depthwise layers of config 2 at batch 256
// (102.8 MB in; 102.8 MB and 25.7 MB out) and the pointwise layer of config 1 (51.4 MB in, 25.7 MB out).
// Four buffer pairs are used in turn (822 MB for the largest case: more than the 256 MB of last-level cache), one
// event pair brackets 100 launches, the figure printed is the median of 8 such regions after 2 discarded ones.
// Last, the approach to the settled rate from a cold start: region by region, with the shader clock read by a
// one-wave probe kernel behind every region (a memory-bound kernel's time should not follow the shader clock; this
// shows whether the slower first milliseconds of a run do).
//
// Build: hipcc --offload-arch=gfx950 -O3 -std=c++17 hbm_ceiling.hip -o hbm_ceiling   (python -m pulp_nn_amd.build does it)
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <unistd.h>
#include <algorithm>
#include <vector>

#define CK(x)                                                                      \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);        \
      exit(1);                                                                     \
    }                                                                              \
  } while (0)

typedef int v4i __attribute__((ext_vector_type(4)));

// a workgroup of 256 lanes moves `per` consecutive 4 KB blocks; n16 = number of 16-byte pieces
template <bool NT>
__global__ __launch_bounds__(256) void copy_kernel(const v4i *__restrict__ in, v4i *__restrict__ out, size_t n_in, size_t n_out,
                                                   int per)
{
  const size_t base = (size_t)blockIdx.x * per * 256 + threadIdx.x;
  for (int i = 0; i < per; i++) {
    const size_t idx = base + (size_t)i * 256;
    if (idx < n_in) {
      const v4i v = NT ? __builtin_nontemporal_load(in + idx) : in[idx];
      if (idx < n_out) {
        if (NT) __builtin_nontemporal_store(v, out + idx);
        else out[idx] = v;
      } else if (v.x == 0x12345 && v.y == 0x6789a) {
        out[0] = v;  // never: keeps the load of the part that has no output
      }
    }
  }
}

__global__ __launch_bounds__(256) void read_kernel(const v4i *__restrict__ in, int *out, size_t n16, int per)
{
  const size_t base = (size_t)blockIdx.x * per * 256 + threadIdx.x;
  int acc = 0;
  for (int i = 0; i < per; i++) {
    const size_t idx = base + (size_t)i * 256;
    if (idx < n16) {
      const v4i v = in[idx];
      acc += v.x ^ v.y ^ v.z ^ v.w;
    }
  }
  if (acc == 0x12345) out[0] = acc;  // never for the fill values used here
}

__global__ __launch_bounds__(256) void write_kernel(v4i *out, size_t n16, int per)
{
  const size_t base = (size_t)blockIdx.x * per * 256 + threadIdx.x;
  for (int i = 0; i < per; i++) {
    const size_t idx = base + (size_t)i * 256;
    if (idx < n16) out[idx] = v4i{(int)idx, 1, 2, 3};
  }
}

// shader clock right now: cycles of the shader counter per tick of the 100 MHz wall clock, over 20 us of one wave
__global__ void clock_probe_kernel(long long *out)
{
  const long long t0 = wall_clock64(), c0 = __builtin_readcyclecounter();
  long long t1 = t0;
  while (t1 - t0 < 2000) t1 = wall_clock64();
  const long long c1 = __builtin_readcyclecounter();
  if (threadIdx.x == 0) {
    out[0] = t1 - t0;
    out[1] = c1 - c0;
  }
}

int main()
{
  struct Case { const char *name; size_t in, out; };
  const Case cases[] = {
      {"depthwise stride 1, 56x56x128 b256", (size_t)256 * 128 * 56 * 56, (size_t)256 * 128 * 56 * 56},
      {"depthwise stride 2, 56x56x128 b256", (size_t)256 * 128 * 56 * 56, (size_t)256 * 128 * 28 * 28},
      {"pointwise 28x28x256 -> 128 b256", (size_t)256 * 28 * 28 * 256, (size_t)256 * 28 * 28 * 128},
  };
  const int NBUF = 4;
  const size_t cap = (size_t)256 * 128 * 56 * 56;
  v4i *din[NBUF], *dout[NBUF];
  for (int i = 0; i < NBUF; i++) {
    CK(hipMalloc(&din[i], cap));
    CK(hipMalloc(&dout[i], cap));
    CK(hipMemset(din[i], i + 1, cap));
    CK(hipMemset(dout[i], 0, cap));
  }
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  auto timeit = [&](const char *name, double bytes, auto launch) {
    const int points = 10, reps = 100;
    std::vector<float> us;
    for (int c = 0; c < points; c++) {
      CK(hipEventRecord(e0, 0));
      for (int q = 0; q < reps; q++) launch(q % NBUF);
      CK(hipEventRecord(e1, 0));
      CK(hipDeviceSynchronize());
      float ms;
      CK(hipEventElapsedTime(&ms, e0, e1));
      us.push_back(ms / reps * 1e3f);
    }
    std::sort(us.begin() + 2, us.end());
    const float med = us[2 + (points - 2) / 2];
    printf("  %-44s %6.1f us  %5.2f TB/s  %5.1f %% of 8 TB/s   (first region %.1f us)\n", name, med, bytes / (med * 1e-6) / 1e12,
           bytes / (med * 1e-6) / 8e12 * 100, us[0]);
  };
  for (const Case &c : cases) {
    printf("%s: %.1f MB in, %.1f MB out\n", c.name, c.in / 1e6, c.out / 1e6);
    const size_t n_in = c.in / 16, n_out = c.out / 16;
    for (int per : {1, 4}) {
      const int grid = (int)((n_in + (size_t)per * 256 - 1) / ((size_t)per * 256));
      const int wgrid = (int)((n_out + (size_t)per * 256 - 1) / ((size_t)per * 256));
      char nm[96];
      snprintf(nm, sizeof nm, "copy, %d x 4 KB per workgroup", per);
      timeit(nm, (double)c.in + c.out, [&](int i) { hipLaunchKernelGGL(copy_kernel<false>, dim3(grid), dim3(256), 0, 0, din[i], dout[i], n_in, n_out, per); });
      snprintf(nm, sizeof nm, "copy nontemporal, %d x 4 KB per workgroup", per);
      timeit(nm, (double)c.in + c.out, [&](int i) { hipLaunchKernelGGL(copy_kernel<true>, dim3(grid), dim3(256), 0, 0, din[i], dout[i], n_in, n_out, per); });
      snprintf(nm, sizeof nm, "read only, %d x 4 KB per workgroup", per);
      timeit(nm, (double)c.in, [&](int i) { hipLaunchKernelGGL(read_kernel, dim3(grid), dim3(256), 0, 0, din[i], (int *)dout[0], n_in, per); });
      snprintf(nm, sizeof nm, "write only, %d x 4 KB per workgroup", per);
      timeit(nm, (double)c.out, [&](int i) { hipLaunchKernelGGL(write_kernel, dim3(wgrid), dim3(256), 0, 0, dout[i], n_out, per); });
    }
    if (c.in == c.out)
      timeit("hipMemcpyAsync device to device", 2.0 * c.in, [&](int i) { CK(hipMemcpyAsync(dout[i], din[i], c.in, hipMemcpyDeviceToDevice, 0)); });
  }
  // The approach to the settled rate: the pointwise layer's copy, 40 regions of 100 launches back to back from a cold
  // start (the GPU idle for 100 ms before), with the shader clock read by a one-wave probe kernel behind every region.
  {
    const Case &c = cases[2];
    const size_t n_in = c.in / 16, n_out = c.out / 16;
    const int grid = (int)((n_in + 255) / 256);
    long long *dprobe, hprobe[2];
    CK(hipMalloc(&dprobe, 16));
    CK(hipDeviceSynchronize());
    usleep(100000);
    printf("approach to the settled rate, %s copy (non-temporal, 1 x 4 KB per workgroup): us per launch (shader MHz behind the region)\n ", c.name);
    double t_ms = 0;
    for (int r = 0; r < 40; r++) {
      CK(hipEventRecord(e0, 0));
      for (int q = 0; q < 100; q++) hipLaunchKernelGGL(copy_kernel<true>, dim3(grid), dim3(256), 0, 0, din[q % NBUF], dout[q % NBUF], n_in, n_out, 1);
      CK(hipEventRecord(e1, 0));
      hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, 0, dprobe);
      CK(hipDeviceSynchronize());
      float ms;
      CK(hipEventElapsedTime(&ms, e0, e1));
      CK(hipMemcpy(hprobe, dprobe, 16, hipMemcpyDeviceToHost));
      t_ms += ms;
      printf(" %.1f (%.0f)", ms * 10.f, hprobe[0] ? 100.0 * hprobe[1] / hprobe[0] : 0.0);
      if (r % 10 == 9) printf("   [%.1f ms]\n ", t_ms);
    }
    printf("\n");
  }
  CK(hipGetLastError());
  return 0;
}
