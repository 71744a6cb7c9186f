// Where the time of the large convolution goes (config 4 of the benchmark: 64 x 64 x 256 -> 63 x 63 x 256, 3 x 3,
// batch 64, 64-bit batch-norm; 299.65 GOP per launch), measured inside igemm_ring_kernel:
//
//   1. the launch-to-launch time under continuous load, as a series: the shader clock of this GPU settles only
//      after some 10 ms of uninterrupted work, so a burst of a few launches and a long run differ;
//   2. per tile round of the persistent workgroups: the wait for the first sub-slice, the main loop, the
//      epilogue (thread 0 of every workgroup stamps the 100 MHz wall clock and the shader cycle counter; the
//      ratio over the main loop is the shader clock while the MFMAs run);
//   3. the same launch with parts taken out (no loads, no fragment reads, one MFMA per sub-slice, no epilogue:
//      results are wrong, only the time counts), each in the settled state;
//   4. the same for two independent workgroups of four waves per compute unit on 256 x 128 tiles.
//
// Build: hipcc --offload-arch=gfx950 -O3 -std=c++17 conv_phases.hip -o ../lib/conv_phases
// (python -m pulp_nn_amd.build does it).  Run without arguments.
#define PULPNN_BN_BITS 64
#define IGR_TRACE
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "igemm.h"
#include "igemm_ring.h"
#include "igemm_patch.h"

#define CK(x)                                                              \
  do {                                                                     \
    hipError_t e_ = (x);                                                   \
    if (e_ != hipSuccess) {                                                \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      exit(1);                                                             \
    }                                                                      \
  } while (0)

static unsigned long long rs = 88172645463325252ull;
static inline unsigned rnd()
{
  rs ^= rs << 13;
  rs ^= rs >> 7;
  rs ^= rs << 17;
  return (unsigned)(rs >> 11);
}

static int g_cus = 256;
static const int B = 64, H = 64, W = 64, Ci = 256, Co = 256, Ho = 63, Wo = 63;
static const double OPS = 2.0 * B * Ho * Wo * Co * 9 * Ci;

// WN = 0: igemm_patch_kernel (4 x 64 pixel patches, an input row staged once per filter row)
template <int WN, int ABL>
static int launch(ConvGeom g, EpiArgs e)
{
  if constexpr (WN == 0) {
    g.tiles_n = (g.N + IGP_BN - 1) / IGP_BN;
    g.rgroups = (g.Ho + 3) / 4;
    g.d_rg = fastdiv_make(g.rgroups);
    g.tiles_total = g.batch * g.rgroups * g.tiles_n;
    g.d_tiles_n = fastdiv_make(g.tiles_n);
    const int unit = 8 * g.tiles_n;
    const int grid = g_cus / unit * unit;
    static bool raised = false;
    if (!raised) {
      CK(hipFuncSetAttribute((const void *)igemm_patch_kernel<EPI_BN, ABL>, hipFuncAttributeMaxDynamicSharedMemorySize, igp_lds_bytes()));
      raised = true;
    }
    hipLaunchKernelGGL((igemm_patch_kernel<EPI_BN, ABL>), dim3(grid), dim3(IGP_THREADS), igp_lds_bytes(), 0, g, e);
    return grid;
  } else {
  typedef IgrShape<WN> S;
  g.tiles_n = (g.N + S::BN - 1) / S::BN;
  g.tiles_total = ((g.M + IGR_BM - 1) / IGR_BM) * g.tiles_n;
  g.d_tiles_n = fastdiv_make(g.tiles_n);
  const int unit = 8 * g.tiles_n;
  const int grid = ((WN == 2 ? 2 : 1) * g_cus) / unit * unit;
  static bool raised = false;
  if (!raised) {
    CK(hipFuncSetAttribute((const void *)igemm_ring_kernel<EPI_BN, WN, ABL>, hipFuncAttributeMaxDynamicSharedMemorySize, S::lds_bytes()));
    raised = true;
  }
  hipLaunchKernelGGL((igemm_ring_kernel<EPI_BN, WN, ABL>), dim3(grid), dim3(S::THREADS), S::lds_bytes(), 0, g, e);
  return grid;
  }
}

template <int WN, int ABL>
static void run(const char *name, const ConvGeom &g, const EpiArgs &e, long long *dtr, bool series)
{
  const int slots = 512 * 64;
  CK(hipMemset(dtr, 0, slots * 8));
  // settled state: 40 points of 50 launches, back to back
  const int points = 40, per = 50;
  std::vector<hipEvent_t> ev(points + 1);
  for (auto &x : ev) CK(hipEventCreate(&x));
  CK(hipEventRecord(ev[0], 0));
  int grid = 0;
  for (int c = 0; c < points; c++) {
    for (int r = 0; r < per; r++) grid = launch<WN, ABL>(g, e);
    CK(hipEventRecord(ev[c + 1], 0));
  }
  CK(hipDeviceSynchronize());
  std::vector<float> us(points);
  for (int c = 0; c < points; c++) {
    float ms;
    CK(hipEventElapsedTime(&ms, ev[c], ev[c + 1]));
    us[c] = ms / per * 1e3f;
  }
  std::vector<float> tail(us.begin() + points / 2, us.end());
  std::sort(tail.begin(), tail.end());
  const float settled = tail[tail.size() / 2];
  // one traced launch right behind the run (the trace costs two clock reads per iteration and wave)
  CK(hipMemcpyToSymbol(HIP_SYMBOL(igr_trace), &dtr, sizeof dtr));
  launch<WN, ABL>(g, e);
  CK(hipDeviceSynchronize());
  long long *null_ptr = nullptr;
  CK(hipMemcpyToSymbol(HIP_SYMBOL(igr_trace), &null_ptr, sizeof null_ptr));
  std::vector<long long> tr(slots);
  CK(hipMemcpy(tr.data(), dtr, slots * 8, hipMemcpyDeviceToHost));
  double first = 0, loop = 0, epi = 0, clk = 0;
  int n = 0;
  for (int w = 0; w < grid; w++)
    for (int r = 1; r < 3; r++) {  // rounds 1 and 2: neither the first tile (weight sums) nor the last, partly filled round
      const long long *q = &tr[(w * 8 + r) * 8];
      if (!q[6]) continue;
      n++;
      first += (q[2] - q[0]) / 100.0;
      loop += (q[4] - q[2]) / 100.0;
      epi += (q[6] - q[4]) / 100.0;
      clk += (double)(q[5] - q[3]) / ((q[4] - q[2]) / 100.0);
    }
  printf("%-44s %7.1f us = %5.3f POP/s | first launches %6.1f us | per tile: wait %4.2f  loop %5.2f  epilogue %4.2f us | clock in loop %4.0f MHz\n",
         name, settled, OPS / (settled * 1e-6) / 1e15, us[0], n ? first / n : 0, n ? loop / n : 0, n ? epi / n : 0, n ? clk / n : 0);
  if (series) {
    printf("    launch-to-launch time over the run, 50 launches per point (us):");
    for (int c = 0; c < points; c += (c < 10 ? 1 : 5)) printf(" %.1f", us[c]);
    printf("\n");
  }
  fflush(stdout);
  for (auto &x : ev) CK(hipEventDestroy(x));
}

int main()
{
  hipDeviceProp_t prop;
  CK(hipGetDeviceProperties(&prop, 0));
  g_cus = prop.multiProcessorCount;
  const size_t nin = (size_t)B * H * W * Ci, nw = (size_t)Co * 9 * Ci, nout = (size_t)B * Ho * Wo * Co;
  std::vector<uint8_t> hin(nin);
  std::vector<int8_t> hw(nw), hb(Co);
  std::vector<bn_t> hk(Co), hl(Co);
  for (auto &v : hin) v = rnd();
  for (auto &v : hw) v = (int8_t)rnd();
  for (auto &v : hb) v = (int8_t)rnd();
  for (int i = 0; i < Co; i++) {
    hk[i] = (1 << 20) + rnd() % (15 << 20);
    hl[i] = (long long)(rnd() % (1u << 31)) * 64 - (1ll << 36);
  }
  uint8_t *din, *dout;
  int8_t *dw, *db;
  bn_t *dk, *dl;
  long long *dtr;
  CK(hipMalloc(&din, nin));
  CK(hipMalloc(&dout, nout));
  CK(hipMalloc(&dw, nw));
  CK(hipMalloc(&db, Co));
  CK(hipMalloc(&dk, 8 * Co));
  CK(hipMalloc(&dl, 8 * Co));
  CK(hipMalloc(&dtr, 512 * 64 * 8));  // 512 workgroups x 8 rounds x 4 stamps of (wall clock, cycle counter)
  CK(hipMemcpy(din, hin.data(), nin, hipMemcpyHostToDevice));
  CK(hipMemcpy(dw, hw.data(), nw, hipMemcpyHostToDevice));
  CK(hipMemcpy(db, hb.data(), Co, hipMemcpyHostToDevice));
  CK(hipMemcpy(dk, hk.data(), 8 * Co, hipMemcpyHostToDevice));
  CK(hipMemcpy(dl, hl.data(), 8 * Co, hipMemcpyHostToDevice));
  ConvGeom g;
  memset(&g, 0, sizeof g);
  g.in = din, g.w = dw, g.bias = db, g.out = dout;
  g.M = B * Ho * Wo, g.N = Co, g.K = 9 * Ci, g.H = H, g.W = W, g.Ci = Ci, g.Ho = Ho, g.Wo = Wo, g.HoWo = Ho * Wo;
  g.kx = g.ky = 3, g.pt = 1, g.pl = 1, g.sx = g.sy = 1, g.in_img = (long long)H * W * Ci, g.batch = B;
  g.vec_store = 1, g.nt = 1;
  g.d_howo = fastdiv_make(g.HoWo), g.d_wo = fastdiv_make(g.Wo);
  g.cpt = Ci / 64, g.d_cpt = fastdiv_make(g.cpt), g.d_kx = fastdiv_make(g.kx);
  EpiArgs e = {dk, dl, 0, 38};
  printf("%s, %d compute units; igemm_ring_kernel on config 4 (random bytes, 64-bit batch-norm), %.2f GOP per launch\n",
         prop.gcnArchName, g_cus, OPS / 1e9);
  printf("columns: settled launch-to-launch time (median of the second half of 2000 launches back to back) | mean of the first 50 launches |\n"
         "         rounds 1 and 2 of a traced launch, mean over the workgroups | shader cycles per wall-clock time over the main loop\n");
  {
    // the two kernels against each other, byte by byte
    std::vector<uint8_t> a(nout), b(nout);
    CK(hipMemset(dout, 0xA5, nout));
    launch<4, 0>(g, e);
    CK(hipDeviceSynchronize());
    CK(hipMemcpy(a.data(), dout, nout, hipMemcpyDeviceToHost));
    CK(hipMemset(dout, 0x5A, nout));
    launch<0, 0>(g, e);
    CK(hipDeviceSynchronize());
    CK(hipGetLastError());
    CK(hipMemcpy(b.data(), dout, nout, hipMemcpyDeviceToHost));
    size_t bad = 0, fb = 0;
    for (size_t i = 0; i < nout; i++)
      if (a[i] != b[i]) {
        if (!bad) fb = i;
        bad++;
      }
    printf("igemm_patch_kernel against igemm_ring_kernel: %zu of %zu output bytes differ", bad, nout);
    if (bad) printf(" (first: pixel %zu channel %zu, %d against %d)", fb / Co, fb % Co, b[fb], a[fb]);
    printf("\n");
    fflush(stdout);
    if (bad) return 1;
  }
  printf("-- 4 x 64 pixel patches, input rows staged once per filter row (igemm_patch_kernel: the library's kernel for this layer) --\n");
  run<0, 0>("complete", g, e, dtr, true);
  run<0, 1>("no loads behind a tile's first two groups", g, e, dtr, false);
  run<0, 4>("no fragment reads in the loop", g, e, dtr, false);
  run<0, 8>("no epilogue", g, e, dtr, false);
  run<0, 32>("activation loads out of range (zeros, no traffic)", g, e, dtr, false);
  run<0, 64>("weight loads out of range", g, e, dtr, false);
  run<0, 96>("all loads out of range", g, e, dtr, false);
  printf("-- 256 consecutive pixels x 256 channels, one sub-slice per tap (igemm_ring_kernel: the library's kernel for other shapes) --\n");
  run<4, 0>("complete", g, e, dtr, true);
  run<4, 1>("no loads behind a tile's first sub-slices", g, e, dtr, false);
  run<4, 4>("no fragment reads in the loop", g, e, dtr, false);
  run<4, 2>("one MFMA per sub-slice instead of 32", g, e, dtr, false);
  run<4, 8>("no epilogue", g, e, dtr, false);
  run<4, 16>("epilogue without its stores", g, e, dtr, false);
  run<4, 13>("MFMAs and xors only (no loads, reads, epilogue)", g, e, dtr, false);
  run<4, 7>("epilogue and loop skeleton only", g, e, dtr, false);
  printf("-- two workgroups of four waves per compute unit, 256 x 128 tiles --\n");
  run<2, 0>("complete", g, e, dtr, true);
  run<2, 1>("no loads behind a tile's first sub-slices", g, e, dtr, false);
  run<2, 8>("no epilogue", g, e, dtr, false);
  return 0;
}
