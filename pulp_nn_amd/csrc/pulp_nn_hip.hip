// C-ABI host layer: the PULP-NN layer functions on MI355X.
//
// Built twice: -DPULPNN_BN_BITS=32 -> libpulpnn_hip32.so, =64 -> libpulpnn_hip64.so,
// mirroring the reference's 32bit/ and 64bit/ trees (same symbol names, k / lambda
// typed int32_t or int64_t).  Each function validates its arguments, picks a
// kernel variant and queues it; nothing is allocated and no state is kept
// besides the per-thread batch count, stream and last error.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#if PULPNN_BN_BITS == 64
#include "../../include/64bit/pulp_nn_kernels.h"
#else
#include "../../include/32bit/pulp_nn_kernels.h"
#endif

#include <algorithm>
#include <atomic>
#include <mutex>

#include "calib.h"
#include "depthwise.h"
#include "dwpw_fused.h"
#include "igemm.h"
#include "igemm_ring.h"
#include "igemm_patch.h"
#include "depthwise_stream.h"
#include "linear_skinny.h"
#include "pool.h"
#include "pw_stream.h"
#include "requant.h"
#include "smallk.h"

namespace {

thread_local unsigned g_batch = 1;
thread_local hipStream_t g_stream = nullptr;
thread_local int g_err = PULP_NN_HIP_OK;
thread_local char g_errmsg[256] = "";

void set_error(int code, const char *fn, const char *msg)
{
  g_err = code;
  snprintf(g_errmsg, sizeof g_errmsg, "%s: %s", fn, msg);
}

#define REQUIRE(cond, code, msg)        \
  do {                                  \
    if (!(cond)) {                      \
      set_error((code), __func__, msg); \
      return;                           \
    }                                   \
  } while (0)

void check_launch(const char *fn)
{
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) set_error(PULP_NN_HIP_ERR_RUNTIME, fn, hipGetErrorString(e));
}

inline bool aligned(const void *p, unsigned a) { return ((uintptr_t)p & (a - 1)) == 0; }

// Shift as the reference's quantisers see it, plus range validation.
// Returns false if the shift would be undefined behaviour in the reference.
bool epi_args(int mode, const bn_t *k, const bn_t *lambda, uint16_t out_mult, int out_shift_param, EpiArgs *e)
{
  e->k = k;
  e->lambda = lambda;
  e->mult = (int)(int16_t)out_mult;
  if (mode == EPI_RAW) {
    e->shift = out_shift_param;  // used as written: sum >> out_shift
    return e->shift >= 0 && e->shift < 32;
  }
  e->shift = (int)(int8_t)out_shift_param;  // the quantiser functions take int8_t
  const int lim = (mode == EPI_BN) ? PULPNN_BN_BITS : 32;
  if (mode == EPI_BN && (!k || !lambda)) return false;
  return e->shift >= 0 && e->shift < lim;
}

// Compute units of the current device.  Cached per process; concurrent first calls compute the
// same value, so a relaxed atomic is enough.
int num_cus()
{
  static std::atomic<int> cached{0};
  int n = cached.load(std::memory_order_relaxed);
  if (!n) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) n = p.multiProcessorCount;
    if (n <= 0) n = 256;
    cached.store(n, std::memory_order_relaxed);
  }
  return n;
}

// ---- implicit GEMM dispatch -------------------------------------------------

// launch-constant divisions of the tiled kernels (call after tiles_n is known)
void conv_geom_divs(ConvGeom &g)
{
  g.d_howo = fastdiv_make((unsigned)g.HoWo);
  g.d_wo = fastdiv_make((unsigned)g.Wo);
  g.d_tiles_n = fastdiv_make((unsigned)g.tiles_n);
  g.batch = (g.M + g.HoWo - 1) / g.HoWo;
  g.ci_shift = 0;
  while ((1 << (g.ci_shift + 1)) <= g.Ci) g.ci_shift++;
  g.rkx = 65536 / g.kx + 1;
}

template <int TN, int WM_, int WN_, int GATHER, int TM = 4, int ONEPASS = 0>
void launch_igemm_mode(int mode, ConvGeom &g, const EpiArgs &e, hipStream_t s)
{
  constexpr int BM = 16 * TM * WM_, BN = 16 * TN * WN_;
  const int tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  g.tiles_total = tiles_m * g.tiles_n;
  conv_geom_divs(g);
  g.vec_store = (g.N % (4 * TN) == 0) && aligned(g.out, 4 * TN);
  // default store policy: the tiled kernel is not bound by HBM, its 16-byte pieces would reach HBM
  // uncombined with the streaming policy (1.36 x the bytes), and the next layer finds the output in cache
  g.nt = 0;
  dim3 grid(g.tiles_total), block(64 * WM_ * WN_);
  switch (mode) {
    case EPI_BN: hipLaunchKernelGGL((igemm_kernel<TN, WM_, WN_, GATHER, EPI_BN, TM, ONEPASS>), grid, block, 0, s, g, e); break;
    case EPI_MULT: hipLaunchKernelGGL((igemm_kernel<TN, WM_, WN_, GATHER, EPI_MULT, TM, ONEPASS>), grid, block, 0, s, g, e); break;
    case EPI_RAW: hipLaunchKernelGGL((igemm_kernel<TN, WM_, WN_, GATHER, EPI_RAW, TM, ONEPASS>), grid, block, 0, s, g, e); break;
    default: hipLaunchKernelGGL((igemm_kernel<TN, WM_, WN_, GATHER, EPI_OUT32, TM, ONEPASS>), grid, block, 0, s, g, e); break;
  }
}

// Raises a kernel's dynamic-LDS limit above the default 64 KB, once per process and kernel.
template <auto KERN>
bool raise_lds_limit(size_t lds)
{
  static std::mutex mu;
  static std::atomic<size_t> limit{65536};
  if (lds > limit.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> lock(mu);
    if (lds > limit.load(std::memory_order_relaxed)) {
      if (hipFuncSetAttribute((const void *)KERN, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
      limit.store(lds, std::memory_order_release);
    }
  }
  return true;
}

// 256 x 256 tiles of persistent workgroups fed by LDS-direct loads (igemm_ring.h).  Returns false if the shape
// does not qualify or the kernel cannot be launched (the caller then uses the tiled kernel).
bool launch_igemm_ring(int mode, ConvGeom &g, const EpiArgs &e, hipStream_t s)
{
  typedef IgrShape<4> S;
  // K: at least as many sub-slices as ring stages; below 2^16, so that accumulator and correction term each
  // fit 32 bits (the epilogue adds them in 64-bit arithmetic in the 64-bit build)
  if (g.Ci % 64 || g.K < 64 * S::NS || g.K >= 65536 || g.N % 16 || !aligned(g.out, 16) || mode == EPI_OUT32) return false;
  g.tiles_n = (g.N + S::BN - 1) / S::BN;
  g.tiles_total = ((g.M + IGR_BM - 1) / IGR_BM) * g.tiles_n;
  // the grid: a multiple of 8 * tiles_n workgroups (a workgroup keeps its channel range, an XCD gets whole
  // pixel tiles), at most one per compute unit and no more than there are tiles
  const int unit = 8 * g.tiles_n;
  const int grid_n = (int)(std::min<long long>(num_cus(), g.tiles_total) / unit) * unit;
  if (grid_n <= 0) return false;
  conv_geom_divs(g);
  g.cpt = g.Ci / 64;
  g.d_cpt = fastdiv_make((unsigned)g.cpt);
  g.d_kx = fastdiv_make((unsigned)g.kx);
  g.vec_store = 1;
  g.nt = (long long)g.M * g.N >= PULPNN_NT_BYTES;
  const size_t lds = (size_t)S::lds_bytes();
  const dim3 grid(grid_n), block(S::THREADS);
  switch (mode) {
    case EPI_BN:
      if (!raise_lds_limit<igemm_ring_kernel<EPI_BN, 4>>(lds)) return false;
      hipLaunchKernelGGL((igemm_ring_kernel<EPI_BN, 4>), grid, block, lds, s, g, e);
      break;
    case EPI_MULT:
      if (!raise_lds_limit<igemm_ring_kernel<EPI_MULT, 4>>(lds)) return false;
      hipLaunchKernelGGL((igemm_ring_kernel<EPI_MULT, 4>), grid, block, lds, s, g, e);
      break;
    default:
      if (!raise_lds_limit<igemm_ring_kernel<EPI_RAW, 4>>(lds)) return false;
      hipLaunchKernelGGL((igemm_ring_kernel<EPI_RAW, 4>), grid, block, lds, s, g, e);
      break;
  }
  return true;
}

// 4-row x 64-column output patches whose input rows are staged once per filter row (igemm_patch.h): 3-wide
// stride-1 filters on images of 57 to 64 output columns.  Returns false if the shape does not qualify.
bool launch_igemm_patch(int mode, ConvGeom &g, const EpiArgs &e, hipStream_t s)
{
  if (g.kx != 3 || g.sx != 1 || g.sy != 1 || g.pl > 1 || g.Wo > 64 || g.ky > 31) return false;
  if (g.Ci % 64 || g.ky * (g.Ci / 64) < 2 || g.K >= 65536 || g.N % 16 || !aligned(g.out, 16) || mode == EPI_OUT32) return false;
  if (g.M % g.HoWo) return false;  // whole images
  // pixels wanted against pixels computed (whole patches): at least nine tenths
  const int rgroups = (g.Ho + 3) / 4;
  if ((long long)g.Ho * g.Wo * 10 < (long long)rgroups * 4 * 64 * 9) return false;
  g.tiles_n = (g.N + IGP_BN - 1) / IGP_BN;
  conv_geom_divs(g);
  g.rgroups = rgroups;
  g.d_rg = fastdiv_make((unsigned)rgroups);
  const long long tiles = (long long)g.batch * rgroups * g.tiles_n;
  if (tiles > 0x7fffffffLL) return false;
  g.tiles_total = (int)tiles;
  const int unit = 8 * g.tiles_n;
  const int grid_n = (int)(std::min<long long>(num_cus(), g.tiles_total) / unit) * unit;
  if (grid_n <= 0) return false;
  g.cpt = g.Ci / 64;
  g.d_cpt = fastdiv_make((unsigned)g.cpt);
  g.d_kx = fastdiv_make((unsigned)g.kx);
  g.vec_store = 1;
  g.nt = (long long)g.M * g.N >= PULPNN_NT_BYTES;
  const size_t lds = (size_t)igp_lds_bytes();
  const dim3 grid(grid_n), block(IGP_THREADS);
  switch (mode) {
    case EPI_BN:
      if (!raise_lds_limit<igemm_patch_kernel<EPI_BN>>(lds)) return false;
      hipLaunchKernelGGL((igemm_patch_kernel<EPI_BN>), grid, block, lds, s, g, e);
      break;
    case EPI_MULT:
      if (!raise_lds_limit<igemm_patch_kernel<EPI_MULT>>(lds)) return false;
      hipLaunchKernelGGL((igemm_patch_kernel<EPI_MULT>), grid, block, lds, s, g, e);
      break;
    default:
      if (!raise_lds_limit<igemm_patch_kernel<EPI_RAW>>(lds)) return false;
      hipLaunchKernelGGL((igemm_patch_kernel<EPI_RAW>), grid, block, lds, s, g, e);
      break;
  }
  return true;
}

// 128 px x 64 ch tiles, for layers too small to fill the machine with larger ones.  With at most five
// K slices (K <= 320) a tile's whole K extent fits in LDS and is fetched in one go.  Eight waves of 32 x 32 per tile
// rather than four of 64 x 32: these layers are a chain of latencies (gather, stage, multiply, store), and with twice
// the waves every link is issued in half the time (config 0: 7.0 -> 6.6 us).
template <int GATHER>
void launch_igemm_small(int mode, ConvGeom &g, const EpiArgs &e, hipStream_t s)
{
  if (GATHER != GATHER_BYTES && g.K <= 5 * IGEMM_BK) launch_igemm_mode<2, 4, 2, GATHER, 2, 5>(mode, g, e, s);
  else launch_igemm_mode<2, 4, 2, GATHER, 2>(mode, g, e, s);
}

template <int GATHER>
void launch_igemm_tile(int mode, ConvGeom &g, const EpiArgs &e, hipStream_t s)
{
  // 256 px x 256 ch with 16 waves when there are at least two such tiles per CU: half the
  // L2 -> LDS bytes per multiply of the 128 x 128 tile
  const long long big_tiles = (long long)((g.M + 255) / 256) * ((g.N + 255) / 256);
  if (GATHER == GATHER_UNIFORM && g.N > 128 && big_tiles >= 2 * num_cus()) {
    // operands go HBM/L2 -> LDS without passing through registers, persistent workgroups
    if (launch_igemm_patch(mode, g, e, s)) return;
    if (launch_igemm_ring(mode, g, e, s)) return;
    launch_igemm_mode<4, 4, 4, GATHER>(mode, g, e, s);
  } else
  // 128 px x 64 ch while 128 x 128 tiles would give a CU at most one workgroup: twice the workgroups to
  // hide each other's latency (such layers are a few K slices long)
  if (g.N > 64 && (long long)((g.M + 127) / 128) * ((g.N + 127) / 128) <= num_cus()) launch_igemm_small<GATHER>(mode, g, e, s);
  else
  if (g.N > 64) launch_igemm_mode<4, 2, 2, GATHER>(mode, g, e, s);       // 128 px x 128 ch
  else if (g.N > 32 && (g.M + 255) / 256 < 2 * num_cus()) launch_igemm_small<GATHER>(mode, g, e, s);  // 128 px x 64 ch: more workgroups
  else if (g.N > 32) launch_igemm_mode<4, 4, 1, GATHER>(mode, g, e, s);  // 256 px x 64 ch
  else if (g.N > 16) launch_igemm_mode<2, 4, 1, GATHER>(mode, g, e, s);  // 256 px x 32 ch
  else launch_igemm_mode<1, 4, 1, GATHER>(mode, g, e, s);                // 256 px x 16 ch
}

void launch_igemm(int mode, ConvGeom &g, const EpiArgs &e, hipStream_t s)
{
  const bool chunk16 = (g.Ci % 16 == 0) && aligned(g.in, 16) && aligned(g.w, 16);
  // scalar tap walk + range-checked buffer loads: whole K slices inside one tap, one bit
  // per tap in a 32-bit mask, 32-bit byte offsets
  const long long batch = (g.M + g.HoWo - 1) / g.HoWo;
  const bool uniform = chunk16 && (g.Ci % 64 == 0) && g.kx * g.ky <= 32 &&
                       batch * g.in_img + (long long)(g.pt * g.W + g.pl) * g.Ci < 0x7fffffffLL &&
                       (long long)g.N * g.K < 0x7fffffffLL;
  // 16 or 32 input channels: two or four whole taps per K slice, same buffer loads (one bit per tap up to
  // the end of the last slice must fit the 32-bit mask)
  const bool subtap = chunk16 && (g.Ci == 16 || g.Ci == 32) && g.kx * g.ky + 64 / g.Ci <= 32 && g.kx <= 32 &&
                      batch * g.in_img + (long long)(g.pt * g.W + g.pl) * g.Ci + (long long)(g.ky * g.W + g.kx) * g.Ci < 0x7fffffffLL &&
                      (long long)g.N * g.K + 64 < 0x7fffffffLL;
  if (uniform) launch_igemm_tile<GATHER_UNIFORM>(mode, g, e, s);
  else if (subtap) launch_igemm_tile<GATHER_SUBTAP>(mode, g, e, s);
  else if (chunk16) launch_igemm_tile<GATHER_CHUNK16>(mode, g, e, s);
  else launch_igemm_tile<GATHER_BYTES>(mode, g, e, s);
}

// Direct (vector ALU) convolution for small filters and at most 32 channels.  rows: the filter
// has at most 3 rows of at most 12 bytes and is gathered a row at a time (smallk_rows_kernel);
// otherwise it is at most 32 bytes long and gathered byte by byte (smallk_conv_kernel).
template <int NCH>
void launch_smallk(int mode, bool rows, ConvGeom &g, const EpiArgs &e, hipStream_t s)
{
  g.vec_store = (g.N == NCH) && aligned(g.out, 16);
  g.nt = (long long)g.M * g.N >= PULPNN_NT_BYTES;
  dim3 grid((unsigned)((g.M + 255) / 256)), block(256);
  if (rows) {
    // runs of 256 pixels per workgroup: as many as leave every compute unit its eight workgroups
    const long long runs = (g.M + 255) / 256;
    g.tiles_n = (int)std::max<long long>(1, std::min<long long>(8, runs / (8ll * num_cus())));
    g.d_howo = fastdiv_make((unsigned)g.HoWo);
    g.d_wo = fastdiv_make((unsigned)g.Wo);
    grid = dim3((unsigned)((runs + g.tiles_n - 1) / g.tiles_n));
    switch (mode) {
      case EPI_BN: hipLaunchKernelGGL((smallk_rows_kernel<NCH, EPI_BN>), grid, block, 0, s, g, e); break;
      case EPI_MULT: hipLaunchKernelGGL((smallk_rows_kernel<NCH, EPI_MULT>), grid, block, 0, s, g, e); break;
      default: hipLaunchKernelGGL((smallk_rows_kernel<NCH, EPI_RAW>), grid, block, 0, s, g, e); break;
    }
    return;
  }
  switch (mode) {
    case EPI_BN: hipLaunchKernelGGL((smallk_conv_kernel<NCH, EPI_BN>), grid, block, 0, s, g, e); break;
    case EPI_MULT: hipLaunchKernelGGL((smallk_conv_kernel<NCH, EPI_MULT>), grid, block, 0, s, g, e); break;
    default: hipLaunchKernelGGL((smallk_conv_kernel<NCH, EPI_RAW>), grid, block, 0, s, g, e); break;
  }
}


// Launches one instantiation; raises its dynamic-LDS limit above the default 64 KB as needed.
template <auto KERN>
bool launch_pw(const PwGeom &g, const EpiArgs &e, dim3 grid, dim3 block, size_t lds, hipStream_t s)
{
  // (raising the limit twice from two host threads is harmless; the mutex keeps the cached value
  // from running ahead of the attribute)
  static std::mutex mu;
  static std::atomic<size_t> limit{65536};
  if (lds > limit.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> lock(mu);
    if (lds > limit.load(std::memory_order_relaxed)) {
      if (hipFuncSetAttribute((const void *)KERN, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return false;
      }
      limit.store(lds, std::memory_order_release);
    }
  }
  hipLaunchKernelGGL(KERN, grid, block, lds, s, g, e);
  return true;
}

// Two shapes of the streaming kernel: 16 waves taking 16 pixels per step for launches
// with at least three steps for every wave of every CU (more waves in flight hide the
// arithmetic of a step behind the memory traffic of the others), 8 waves taking 32 pixels
// per step otherwise (half the LDS reads per pixel, and the 128-register budget of the
// 16-wave shape is too small for K = 256).
template <int TN, int NP, int KS, int TM, int NW>
bool launch_pw_stream_mode(int mode, const PwGeom &g, const EpiArgs &e, dim3 grid, size_t lds, hipStream_t s)
{
  dim3 block(64 * NW);
  switch (mode) {
    case EPI_BN: return launch_pw<pw_stream_kernel<TN, KS, NP, EPI_BN, false, TM, NW>>(g, e, grid, block, lds, s);
    case EPI_MULT:
      if (e.shift >= 16) return launch_pw<pw_stream_kernel<TN, KS, NP, EPI_MULT, true, TM, NW>>(g, e, grid, block, lds, s);
      return launch_pw<pw_stream_kernel<TN, KS, NP, EPI_MULT, false, TM, NW>>(g, e, grid, block, lds, s);
    default: return launch_pw<pw_stream_kernel<TN, KS, NP, EPI_RAW, false, TM, NW>>(g, e, grid, block, lds, s);
  }
}

template <int TN, int NP>
bool launch_pw_stream_ks(int mode, int ks, bool wide, const PwGeom &g, const EpiArgs &e, dim3 grid, size_t lds,
                         hipStream_t s)
{
  if (ks == 1) {
    if (wide) return launch_pw_stream_mode<TN, NP, 1, 1, 16>(mode, g, e, grid, lds, s);
    return launch_pw_stream_mode<TN, NP, 1, 2, 8>(mode, g, e, grid, lds, s);
  } else if (ks == 2) {
    if (wide) return launch_pw_stream_mode<TN, NP, 2, 1, 16>(mode, g, e, grid, lds, s);
    return launch_pw_stream_mode<TN, NP, 2, 2, 8>(mode, g, e, grid, lds, s);
  } else {
    return launch_pw_stream_mode<TN, NP, 4, 2, 8>(mode, g, e, grid, lds, s);
  }
}

// Weights-stationary streaming path: a GEMM whose rows are contiguous K-byte pixels,
// whose weight matrix (at most 256 x 256) fits in LDS and whose channel count is one
// of 16, 32, 64, 128, 192, 256 (every lane then owns real channels and stores whole
// vectors).  Returns false if the shape does not qualify (the caller then uses the
// tiled kernel).
bool try_pw_stream(int mode, const uint8_t *in, const int8_t *w, const int8_t *bias, void *out, long long M, int N,
                   int K, const EpiArgs &e, hipStream_t s)
{
  if (K > 256 || (K % 16) || !aligned(in, 16) || !aligned(w, 16) || !aligned(out, 16) || M < 2048) return false;
  if (!(N == 16 || N == 32 || N == 64 || N == 128 || N == 192 || N == 256)) return false;
  if (mode == EPI_OUT32) return false;
  const int tn = N == 16 ? 1 : (N == 32 ? 2 : 4);
  const int np = N / (16 * tn);
  const int ks = K <= 64 ? 1 : (K <= 128 ? 2 : 4);
  PwGeom g;
  g.in = in;
  g.w = w;
  g.bias = bias;
  g.out = out;
  g.M = (int)M;
  g.N = N;
  g.K = K;
  g.units = (int)((M + 15) / 16);
  g.nt = M * N >= PULPNN_NT_BYTES;
  const bool wide = ks <= 2 && g.units >= 3 * 16 * num_cus();
  const int nw = wide ? 16 : 8, tm = wide ? 1 : 2;
  const int lds = pw_lds_bytes(tn, ks, np, mode == EPI_BN, nw, tm);
  if (lds > 160 * 1024 - 512) return false;  // 512: static LDS of the kernel
  // Persistent grid: one workgroup per CU (the weights are staged once per CU), fewer
  // when there are not two 16-pixel units for every wave.
  int blocks = num_cus();
  const int need = (g.units + 2 * nw - 1) / (2 * nw);
  if (blocks > need) blocks = need;
  // a launch that would leave more than half of the CUs without a workgroup is better off tiled:
  // every CU takes part there, and staging the weights per workgroup no longer pays
  if (2 * need < num_cus()) return false;
  dim3 grid(blocks);
  // (false also if the kernel's LDS limit cannot be raised: the caller then uses the tiled kernel)
  if (tn == 1) return launch_pw_stream_ks<1, 1>(mode, ks, wide, g, e, grid, lds, s);
  if (tn == 2) return launch_pw_stream_ks<2, 1>(mode, ks, wide, g, e, grid, lds, s);
  if (np == 1) return launch_pw_stream_ks<4, 1>(mode, ks, wide, g, e, grid, lds, s);
  if (np == 2) return launch_pw_stream_ks<4, 2>(mode, ks, wide, g, e, grid, lds, s);
  if (np == 3) return launch_pw_stream_ks<4, 3>(mode, ks, wide, g, e, grid, lds, s);
  return launch_pw_stream_ks<4, 4>(mode, ks, wide, g, e, grid, lds, s);
}

// Shared body of the six convolution entry points.
void conv_common(const char *fn, bool pointwise, const uint8_t *in, const int8_t *bias, uint8_t *out,
                 const int8_t *w, bn_t *k, bn_t *lambda, uint16_t out_mult, uint16_t out_shift,
                 uint16_t dim_in_x, uint16_t dim_in_y, uint16_t ch_in, uint16_t dim_out_x, uint16_t dim_out_y,
                 uint16_t ch_out, uint16_t kx, uint16_t ky, uint16_t pt, uint16_t pl, uint16_t sx, uint16_t sy,
                 int flag_relu, int flag_batch_norm)
{
  if (!in || !out || !w) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "null activation or weight pointer");
  if (!dim_in_x || !dim_in_y || !ch_in || !dim_out_x || !dim_out_y || !ch_out)
    return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "zero dimension");
  if (pointwise) {
    // pulp_nn_pointwise_HoWo_parallel.c:103 reads pixel (y, x) of the input for output (y, x)
    kx = ky = 1;
    pt = pl = 0;
    sx = sy = 1;
    if (dim_out_x > dim_in_x || dim_out_y > dim_in_y)
      return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "pointwise output larger than input");
  } else if (!kx || !ky || !sx || !sy) {
    return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "zero kernel size or stride");
  }
  const int mode = epi_mode(flag_relu, flag_batch_norm);
  EpiArgs e;
  if (!epi_args(mode, k, lambda, out_mult, out_shift, &e))
    return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "out_shift out of range or null k/lambda");
  const long long M = (long long)g_batch * dim_out_x * dim_out_y;
  if (M > 0x7fffffffLL) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "batch too large");
  if (kx == 1 && ky == 1 && sx == 1 && sy == 1 && pt == 0 && pl == 0 && dim_out_x == dim_in_x &&
      dim_out_y == dim_in_y && try_pw_stream(mode, in, w, bias, out, M, ch_out, ch_in, e, g_stream)) {
    check_launch(fn);
    return;
  }
  ConvGeom g;
  g.in = in;
  g.w = w;
  g.bias = bias;
  g.out = out;
  g.M = (int)M;
  g.N = ch_out;
  g.K = (int)kx * ky * ch_in;
  g.H = dim_in_y;
  g.W = dim_in_x;
  g.Ci = ch_in;
  g.Ho = dim_out_y;
  g.Wo = dim_out_x;
  g.HoWo = (int)dim_out_x * dim_out_y;
  g.kx = kx;
  g.ky = ky;
  g.pt = pt;
  g.pl = pl;
  g.sx = sx;
  g.sy = sy;
  g.in_img = (long long)dim_in_x * dim_in_y * ch_in;
  // a filter row is kx * ch_in contiguous input bytes: three aligned dwords cover it if it is at
  // most 9 bytes long, or 12 with rows that start on a dword
  const int row_bytes = (int)kx * ch_in;
  const long long batch = (g.M + g.HoWo - 1) / g.HoWo;
  const bool rows = ky <= 3 && (row_bytes <= 9 || (row_bytes <= 12 && ch_in % 4 == 0)) && aligned(g.in, 4) &&
                    batch * g.in_img < 0x7ffffff0LL;
  if ((rows || g.K <= 4 * SMALLK_KD) && g.N <= 32) {
    if (g.N <= 16) launch_smallk<16>(mode, rows, g, e, g_stream);
    else launch_smallk<32>(mode, rows, g, e, g_stream);
  } else {
    launch_igemm(mode, g, e, g_stream);
  }
  check_launch(fn);
}

void linear_common(const char *fn, int mode, const uint8_t *in, const int8_t *bias, void *out, const int8_t *w,
                   const EpiArgs &e, uint16_t dim_vec, uint16_t num_o_neurons, int rows)
{
  if (!in || !out || !w) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "null pointer");
  if (!dim_vec || !num_o_neurons) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "zero dimension");
  // few rows: a workgroup per 16 neurons streams their weights once, no staging and no K-slice barriers
  if (rows <= 256 && dim_vec % 16 == 0 && aligned(in, 16) && aligned(w, 16) && aligned(out, 4)) {
    const int rblocks = (rows + 63) / 64, ngroups = (num_o_neurons + 15) / 16;
    // K in four parts and a workgroup per block of rows while that still leaves CUs without work
    const bool spread = ngroups * rblocks <= 2 * num_cus();
    const int kparts = spread ? 4 : (rblocks == 1 ? 4 : (rblocks == 2 ? 2 : 1));
    SkinnyGeom sg = {in, w, bias, out, rows, (int)num_o_neurons, (int)dim_vec, kparts};
    const dim3 grid(ngroups, spread ? rblocks : 1), block(256);
    switch (mode) {
      case EPI_BN: hipLaunchKernelGGL(linear_skinny_kernel<EPI_BN>, grid, block, 0, g_stream, sg, e); break;
      case EPI_MULT: hipLaunchKernelGGL(linear_skinny_kernel<EPI_MULT>, grid, block, 0, g_stream, sg, e); break;
      case EPI_RAW: hipLaunchKernelGGL(linear_skinny_kernel<EPI_RAW>, grid, block, 0, g_stream, sg, e); break;
      default: hipLaunchKernelGGL(linear_skinny_kernel<EPI_OUT32>, grid, block, 0, g_stream, sg, e); break;
    }
    check_launch(fn);
    return;
  }
  ConvGeom g;
  g.in = in;
  g.w = w;
  g.bias = bias;
  g.out = out;
  g.M = rows;
  g.N = num_o_neurons;
  g.K = dim_vec;
  g.H = g.W = 1;
  g.Ci = dim_vec;
  g.Ho = g.Wo = g.HoWo = 1;
  g.kx = g.ky = 1;
  g.pt = g.pl = 0;
  g.sx = g.sy = 1;
  g.in_img = dim_vec;
  launch_igemm(mode, g, e, g_stream);
  check_launch(fn);
}

// ---- depthwise dispatch -------------------------------------------------------

void depthwise_common(const char *fn, const uint8_t *in, const int8_t *bias, uint8_t *out, const int8_t *wt,
                      bn_t *k, bn_t *lambda, uint16_t out_mult, int out_shift, int W, int H, int Wo, int Ho, int CH,
                      int kx, int ky, int pt, int pl, int sx, int sy, int mode, bool hwc_in = false)
{
  if (!in || !out || !wt) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "null activation or weight pointer");
  if (W <= 0 || H <= 0 || Wo <= 0 || Ho <= 0 || CH <= 0 || kx <= 0 || ky <= 0 || sx <= 0 || sy <= 0)
    return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "zero dimension");
  EpiArgs e;
  if (!epi_args(mode, k, lambda, out_mult, out_shift, &e))
    return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "out_shift out of range or null k/lambda");
  // the accumulators of these kernels fit easily; guard the i32 sum anyway
  if ((long long)kx * ky > 4096) return set_error(PULP_NN_HIP_ERR_UNSUPPORTED, fn, "kernel too large");

  DwGeom g;
  g.in = in;
  g.wt = wt;
  g.bias = bias;
  g.out = out;
  g.B = (int)g_batch;
  g.CH = CH;
  g.H = H;
  g.W = W;
  g.Ho = Ho;
  g.Wo = Wo;
  g.kx = kx;
  g.ky = ky;
  g.pt = pt;
  g.pl = pl;
  g.sx = sx;
  g.sy = sy;
  const bool fast = kx == 3 && ky == 3 && sx == sy && (sx == 1 || sx == 2) && (pl == 0 || pl == 1);
  // linear variant: LDS rows are the image rows themselves (W / 4 dwords, no padding)
  const bool lin = fast && (W % 4 == 0) && aligned(in, 16) && W / 4 * 3 <= 255;
  g.LP = pl > 4 ? ((pl + 3) & ~3) : 4;
  int need_bytes;  // bytes of an LDS row the compute phase may touch
  if (fast) {
    const int xgroups = (Wo + 3) / 4;
    const int ns = ((4 - pl) + 3 * sx + 2) / 4 + 1;
    need_bytes = 4 * (g.LP / 4 - 1 + (xgroups - 1) * sx + ns);
  } else {
    need_bytes = g.LP - pl + (Wo - 1) * sx + kx;
  }
  const int img_bytes = g.LP + W + 1;
  g.LWD = ((need_bytes > img_bytes ? need_bytes : img_bytes) + 3) / 4;
  if (lin) {
    g.LP = 0;
    g.LWD = W / 4;
  }
  int max_csd = 255;  // 64 channels x 255 dwords = 63.75 KiB of LDS
  // Whole 64-channel groups (the LDS-direct staging of dw3x3_lin_kernel): bands of under 40 KiB, so that four
  // workgroups share a compute unit and the loads of one are covered by the arithmetic of the others; not when
  // that would leave fewer than 6 (stride 2: 4) output rows per band (ky - sy more input rows are staged per
  // band than it consumes alone).
  const bool lin_dma_ok = lin && CH % DW_CG == 0 && Wo % 4 == 0 && aligned(out, 4) &&
                          (long long)g_batch * CH * H * W < 0x7fffffffLL;
  if (lin_dma_ok && (156 / g.LWD - ky) / sy + 1 >= (sx == 1 ? 6 : 4)) max_csd = 156;
  int nr_max = max_csd / g.LWD;
  if (nr_max < ky) return set_error(PULP_NN_HIP_ERR_UNSUPPORTED, fn, "image too wide for the LDS tile");
  int rb_max = (nr_max - ky) / sy + 1;
  if (rb_max > Ho) rb_max = Ho;
  g.bands = (Ho + rb_max - 1) / rb_max;
  g.RB = (Ho + g.bands - 1) / g.bands;
  g.bands = (Ho + g.RB - 1) / g.RB;
  g.NR = (g.RB - 1) * sy + ky;
  g.CSD = (g.NR * g.LWD) | 1;
  g.CHR = CH;
  g.planes = (long long)g.B * CH;
  if (lin && CH < DW_CG && DW_CG % CH == 0 && CH % 4 == 0) {
    // fewer than 64 channels: 64 / CH images share a workgroup (one plane per lane)
    g.CH = DW_CG;
    g.B = (int)((g.planes + DW_CG - 1) / DW_CG);
  }
  g.cgroups = (g.CH + DW_CG - 1) / DW_CG;
  const long long total = (long long)g.B * g.bands * g.cgroups;
  if (total > 0x7fffffffLL) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "batch too large");
  g.total = (int)total;
  g.inc_dw = 256 % g.LWD;
  const int carry = 256 / g.LWD;
  g.inc_row = carry % g.NR;
  g.inc_c = carry / g.NR;
  g.in_align4 = aligned(in, 4) && (W % 4 == 0);
  g.out_vec4 = aligned(out, 4) && (CH % 4 == 0);
  const size_t lds = (size_t)DW_CG * g.CSD * 4;
  dim3 grid(g.total), block(256);
#define DW_LAUNCH(KERNEL)                                                                   \
  switch (mode) {                                                                           \
    case EPI_BN: hipLaunchKernelGGL((KERNEL<EPI_BN>), grid, block, lds, g_stream, g, e); break;     \
    case EPI_MULT: hipLaunchKernelGGL((KERNEL<EPI_MULT>), grid, block, lds, g_stream, g, e); break; \
    default: hipLaunchKernelGGL((KERNEL<EPI_RAW>), grid, block, lds, g_stream, g, e); break;        \
  }
#define DW3(S, PL, M) dw3x3_kernel<S, PL, M>
  // small square planes, padding 1: one plane per lane, in registers
  const int ho_plane = (H - 1) / sx + 1;
  const bool plane = fast && W == H && pt == 1 && pl == 1 && ((H == 8) || (H == 4 && sx == 1)) && Ho == ho_plane &&
                     Wo == ho_plane && CH % DW_CG == 0 && aligned(in, hwc_in ? 4 : 16) && aligned(out, 4) &&
                     (long long)g.B * g.cgroups <= 0x7fffffffLL;
  // rows of 16, 32 or 64 bytes, padding 1, any height: a few rows of a plane per lane, in registers
  const bool rowsk = !plane && fast && pt == 1 && pl == 1 && (W == 16 || W == 32 || W == 64) && Wo == (W - 1) / sx + 1 &&
                     Ho <= (H - 1) / sy + 1 && CH % 4 == 0 && ((long long)g_batch * CH) % DW_CG == 0 && aligned(in, hwc_in ? 4 : 16) &&
                     aligned(out, 4) && (long long)g_batch * CH / DW_CG * Ho < 0x7fffffffLL;
  // Layers that fill the machine with one workgroup per image and 64 channels (two per compute unit): the plane
  // streamed through LDS, 8 rows of it per request.  Up to 14 groups of 4 output columns, 64 KiB of LDS.  A chunk
  // costs a barrier and a round trip to memory however few rows it holds, so at stride 1 (where the band kernel is
  // within 3 %) only planes of whole chunks take this kernel: 56 rows do, the 58 pre-padded rows of
  // pulp_nn_depthwise_3x3_s1 run 7 % faster in bands.
  const int stream_csd = (2 * DWS_ROWS * (W / 4)) | 1;
  const size_t stream_lds = 4 * ((size_t)DW_CG * stream_csd + 8 * (size_t)(Wo / 4));
  const bool stream = !plane && !rowsk && !hwc_in && lin_dma_ok && Wo / 4 <= 16 - DWS_LOADERS && stream_lds <= 64 * 1024 && DWS_ROWS * W <= 1024 &&
                      (sx == 2 || H % DWS_ROWS == 0) &&
                      (long long)g_batch * (CH / DW_CG) >= 2ll * num_cus();
  if (hwc_in && !plane && !rowsk)
    return set_error(PULP_NN_HIP_ERR_UNSUPPORTED, fn, "no fused kernel for this geometry: use pulp_nn_hip_hwc_to_chw and the CHW entry point");
  if (plane) {
    const dim3 pgrid((unsigned)(((long long)g.B * g.cgroups + DW_REG_WAVES - 1) / DW_REG_WAVES)), pblock(64 * DW_REG_WAVES);
#define DWP_LAYOUT(HW, S, HWC)                                                                                            \
  switch (mode) {                                                                                                         \
    case EPI_BN: hipLaunchKernelGGL((dw3x3_plane_kernel<HW, S, EPI_BN, HWC>), pgrid, pblock, 0, g_stream, g, e); break;     \
    case EPI_MULT: hipLaunchKernelGGL((dw3x3_plane_kernel<HW, S, EPI_MULT, HWC>), pgrid, pblock, 0, g_stream, g, e); break; \
    default: hipLaunchKernelGGL((dw3x3_plane_kernel<HW, S, EPI_RAW, HWC>), pgrid, pblock, 0, g_stream, g, e); break;        \
  }
#define DWP_MODE(HW, S)                      \
  if (hwc_in) { DWP_LAYOUT(HW, S, true) }    \
  else { DWP_LAYOUT(HW, S, false) }
    if (H == 8 && sx == 1) { DWP_MODE(8, 1) }
    else if (H == 8) { DWP_MODE(8, 2) }
    else { DWP_MODE(4, 1) }
#undef DWP_MODE
#undef DWP_LAYOUT
  } else if (rowsk) {
    const long long groups = (long long)g_batch * CH / DW_CG;
#define DWR_LAYOUT(WB, R, S, HWC)                                                                                                \
  {                                                                                                                              \
    const dim3 rgrid((unsigned)((groups * ((Ho + R - 1) / R) + DW_REG_WAVES - 1) / DW_REG_WAVES)), rblock(64 * DW_REG_WAVES);    \
    switch (mode) {                                                                                                              \
      case EPI_BN: hipLaunchKernelGGL((dw3x3_rows_kernel<WB, R, S, EPI_BN, HWC>), rgrid, rblock, 0, g_stream, g, e); break;      \
      case EPI_MULT: hipLaunchKernelGGL((dw3x3_rows_kernel<WB, R, S, EPI_MULT, HWC>), rgrid, rblock, 0, g_stream, g, e); break;  \
      default: hipLaunchKernelGGL((dw3x3_rows_kernel<WB, R, S, EPI_RAW, HWC>), rgrid, rblock, 0, g_stream, g, e); break;         \
    }                                                                                                                            \
  }
#define DWR_MODE(WB, R, S)                       \
  {                                              \
    if (hwc_in) DWR_LAYOUT(WB, R, S, true)       \
    else DWR_LAYOUT(WB, R, S, false)             \
  }
    g.CHR = CH;
    g.planes = (long long)g_batch * CH;
    if (W == 16 && sx == 1) DWR_MODE(16, 8, 1)
    else if (W == 16) DWR_MODE(16, 4, 2)
    else if (W == 32 && sx == 1) DWR_MODE(32, 4, 1)
    else if (W == 32) DWR_MODE(32, 4, 2)
    else if (sx == 1) DWR_MODE(64, 2, 1)
    else DWR_MODE(64, 2, 2)
#undef DWR_MODE
#undef DWR_LAYOUT
  } else if (stream) {
    // whole planes streamed through LDS by loader waves, one workgroup per image and 64 channels
    g.NR = DWS_ROWS;
    g.RB = 2;
    g.CSD = stream_csd;
    g.bands = 1;
    g.total = (int)((long long)g.B * g.cgroups);
    const dim3 sgrid(g.total), sblock(64 * (Wo / 4 + DWS_LOADERS));
#define DWS_MODE(S, PL)                                                                                                  \
  switch (mode) {                                                                                                        \
    case EPI_BN: hipLaunchKernelGGL((dw3x3_stream_kernel<S, PL, EPI_BN>), sgrid, sblock, stream_lds, g_stream, g, e); break;     \
    case EPI_MULT: hipLaunchKernelGGL((dw3x3_stream_kernel<S, PL, EPI_MULT>), sgrid, sblock, stream_lds, g_stream, g, e); break; \
    default: hipLaunchKernelGGL((dw3x3_stream_kernel<S, PL, EPI_RAW>), sgrid, sblock, stream_lds, g_stream, g, e); break;        \
  }
    if (sx == 1 && pl == 1) { DWS_MODE(1, 1) }
    else if (sx == 1) { DWS_MODE(1, 0) }
    else if (pl == 1) { DWS_MODE(2, 1) }
    else { DWS_MODE(2, 0) }
#undef DWS_MODE
  } else if (lin) {
    const bool full = (Wo % 4 == 0) && (g.CH % DW_CG == 0) && (g.planes % DW_CG == 0) && g.out_vec4;
    const size_t ldsl = lds + 16;  // spare dword for masked-off staging writes
    const dim3 block(64 * DW_WAVES);
    const int csd_dma = (((g.NR * g.LWD + 3) & ~3)) | 1;  // room for the last 16-byte piece of a band
#define DW3L_MODE(S, PL, FULL)                                                                                        \
  switch (mode) {                                                                                                     \
    case EPI_BN: hipLaunchKernelGGL((dw3x3_lin_kernel<S, PL, EPI_BN, FULL>), grid, block, ldsl, g_stream, g, e); break;     \
    case EPI_MULT: hipLaunchKernelGGL((dw3x3_lin_kernel<S, PL, EPI_MULT, FULL>), grid, block, ldsl, g_stream, g, e); break; \
    default: hipLaunchKernelGGL((dw3x3_lin_kernel<S, PL, EPI_RAW, FULL>), grid, block, ldsl, g_stream, g, e); break;        \
  }
#define DW3L_DMA(S, PL)                                                                                                     \
  switch (mode) {                                                                                                           \
    case EPI_BN: hipLaunchKernelGGL((dw3x3_lin_kernel<S, PL, EPI_BN, true, true>), grid, block, ldsd, g_stream, g, e); break;     \
    case EPI_MULT: hipLaunchKernelGGL((dw3x3_lin_kernel<S, PL, EPI_MULT, true, true>), grid, block, ldsd, g_stream, g, e); break; \
    default: hipLaunchKernelGGL((dw3x3_lin_kernel<S, PL, EPI_RAW, true, true>), grid, block, ldsd, g_stream, g, e); break;        \
  }
#define DW3L(S, PL)          \
  if (full && lin_dma) {     \
    DW3L_DMA(S, PL)          \
  } else if (full) {         \
    DW3L_MODE(S, PL, true)   \
  } else {                   \
    DW3L_MODE(S, PL, false)  \
  }
    // whole 64-channel groups: the band staged by LDS-direct loads (the channel stride leaves room for the last piece)
    const bool lin_dma = full && lin_dma_ok && g.CHR == CH && g.B == (int)g_batch && DW_CG * (size_t)csd_dma * 4 + 16 <= 64 * 1024;
    const size_t ldsd = DW_CG * (size_t)csd_dma * 4 + 16;
    if (lin_dma) g.CSD = csd_dma;
    if (sx == 1 && pl == 1) { DW3L(1, 1) }
    else if (sx == 1) { DW3L(1, 0) }
    else if (pl == 1) { DW3L(2, 1) }
    else { DW3L(2, 0) }
#undef DW3L
#undef DW3L_DMA
#undef DW3L_MODE
  } else if (fast) {
    if (sx == 1 && pl == 1) { switch (mode) {
      case EPI_BN: hipLaunchKernelGGL((DW3(1, 1, EPI_BN)), grid, block, lds, g_stream, g, e); break;
      case EPI_MULT: hipLaunchKernelGGL((DW3(1, 1, EPI_MULT)), grid, block, lds, g_stream, g, e); break;
      default: hipLaunchKernelGGL((DW3(1, 1, EPI_RAW)), grid, block, lds, g_stream, g, e); break; }
    } else if (sx == 1) { switch (mode) {
      case EPI_BN: hipLaunchKernelGGL((DW3(1, 0, EPI_BN)), grid, block, lds, g_stream, g, e); break;
      case EPI_MULT: hipLaunchKernelGGL((DW3(1, 0, EPI_MULT)), grid, block, lds, g_stream, g, e); break;
      default: hipLaunchKernelGGL((DW3(1, 0, EPI_RAW)), grid, block, lds, g_stream, g, e); break; }
    } else if (pl == 1) { switch (mode) {
      case EPI_BN: hipLaunchKernelGGL((DW3(2, 1, EPI_BN)), grid, block, lds, g_stream, g, e); break;
      case EPI_MULT: hipLaunchKernelGGL((DW3(2, 1, EPI_MULT)), grid, block, lds, g_stream, g, e); break;
      default: hipLaunchKernelGGL((DW3(2, 1, EPI_RAW)), grid, block, lds, g_stream, g, e); break; }
    } else { switch (mode) {
      case EPI_BN: hipLaunchKernelGGL((DW3(2, 0, EPI_BN)), grid, block, lds, g_stream, g, e); break;
      case EPI_MULT: hipLaunchKernelGGL((DW3(2, 0, EPI_MULT)), grid, block, lds, g_stream, g, e); break;
      default: hipLaunchKernelGGL((DW3(2, 0, EPI_RAW)), grid, block, lds, g_stream, g, e); break; }
    }
  } else {
    DW_LAUNCH(dw_generic_kernel)
  }
#undef DW3
#undef DW_LAUNCH
  check_launch(fn);
}

bool pool_geom(const char *fn, PoolGeom *g, uint8_t *in, uint8_t *out, uint16_t W, uint16_t H, uint16_t C,
               uint16_t Wo, uint16_t Ho, uint16_t kx, uint16_t ky, uint16_t pt, uint16_t pb, uint16_t pl,
               uint16_t pr, uint16_t sx, uint16_t sy)
{
  if (!in || !out) { set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "null pointer"); return false; }
  if (!W || !H || !C || !Wo || !Ho || !kx || !ky || !sx || !sy) {
    set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "zero dimension");
    return false;
  }
  g->in = in;
  g->out = out;
  g->B = (int)g_batch;
  g->H = H;
  g->W = W;
  g->C = C;
  g->Ho = Ho;
  g->Wo = Wo;
  g->kx = kx;
  g->ky = ky;
  g->sx = sx;
  g->sy = sy;
  g->pt = pt;
  g->pb = pb;
  g->pl = pl;
  g->pr = pr;
  g->cgroups = (C + 3) / 4;
  g->vec4 = (C % 4 == 0) && aligned(in, 4) && aligned(out, 4);
  g->total = (long long)g->B * Ho * Wo * g->cgroups;
  if ((g->total + 255) / 256 > 0x7fffffffLL) {
    set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "batch too large");
    return false;
  }
  return true;
}

// ---- calibration ---------------------------------------------------------------------

// Device memory of the allocation-free calibration entry point: one partial maximum per
// workgroup.  In host code the array's name only stands for the symbol; its device address
// comes from hipGetSymbolAddress, once per device (every GPU holds its own copy).
#define CALIB_STATIC_SLOTS 8192
static __device__ __align__(256) unsigned long long scratch[CALIB_STATIC_SLOTS];

unsigned long long *static_scratch(const char *fn)
{
  constexpr int MAX_DEV = 64;
  static std::mutex mu;
  static unsigned long long *ptr[MAX_DEV] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) {
    set_error(PULP_NN_HIP_ERR_RUNTIME, fn, "cannot identify the current device");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      set_error(PULP_NN_HIP_ERR_RUNTIME, fn, hipGetErrorString(e));
      return nullptr;
    }
    ptr[dev] = (unsigned long long *)p;
  }
  return ptr[dev];
}

// Shared body of the calibration entry points.  partial: device memory for `slots_avail` partial maxima.
void calib_common(const char *fn, CalibGeom &g, unsigned long long *partial, unsigned long long slots_avail,
                  unsigned long long *result)
{
  if (!g.in || !g.w || !g.k || !result) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "null pointer");
  if (g.W <= 0 || g.H <= 0 || g.Ci <= 0 || g.Wo <= 0 || g.Ho <= 0 || g.Co <= 0 || g.kx <= 0 || g.ky <= 0 || g.sx <= 0 ||
      g.sy <= 0)
    return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "zero dimension");
  // batch * Ho * Wo * Co can pass 2^63 (batch up to 2^31, the dimensions up to 2^16 each): bound it before it is formed
  const unsigned long long per_image = (unsigned long long)g.Ho * g.Wo * g.Co;  // < 2^48
  if ((unsigned long long)g_batch > (1ull << 47) / per_image) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "batch too large");
  g.total = (long long)((unsigned long long)g_batch * per_image);
  g.in_img = (long long)g.H * g.W * g.Ci;
  const unsigned long long slots = ((unsigned long long)g.total + CALIB_CHUNK - 1) / CALIB_CHUNK;
  if (slots > 0x7fffffffull) return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn, "batch too large");
  if (!partial || slots > slots_avail)
    return set_error(PULP_NN_HIP_ERR_ARGUMENT, fn,
                     "layer too large for the partial-maximum buffer (one 8-byte slot per 65536 outputs)");
  hipLaunchKernelGGL(calib_absmax_kernel, dim3((unsigned)slots), dim3(256), 0, g_stream, g, partial);
  hipLaunchKernelGGL(calib_final_kernel, dim3(1), dim3(256), 0, g_stream, partial, (int)slots, result);
  check_launch(fn);
}

CalibGeom calib_conv_geom(const unsigned char *in, const signed char *bias, const signed char *w, const void *k,
                          unsigned short dim_in_x, unsigned short dim_in_y, unsigned short ch_in,
                          unsigned short dim_out_x, unsigned short dim_out_y, unsigned short ch_out,
                          unsigned short kx, unsigned short ky, unsigned short pt, unsigned short pl,
                          unsigned short sx, unsigned short sy)
{
  CalibGeom g = {};
  g.in = in;
  g.w = (const int8_t *)w;
  g.bias = (const int8_t *)bias;
  g.k = (const bn_t *)k;
  g.H = dim_in_y;
  g.W = dim_in_x;
  g.Ci = ch_in;
  g.Ho = dim_out_y;
  g.Wo = dim_out_x;
  g.Co = ch_out;
  g.kx = kx;
  g.ky = ky;
  g.pt = pt;
  g.pl = pl;
  g.sx = sx;
  g.sy = sy;
  return g;
}

}  // namespace

// ---- added entry points -----------------------------------------------------------

// Shader clock right now: cycles of the shader counter against ticks of the 100 MHz wall clock, over 20 us of one
// wave (pulp_nn_hip_clock_probe).
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

extern "C" {

void pulp_nn_hip_set_batch(unsigned n_images)
{
  if (n_images > 0x7fffffffu) return set_error(PULP_NN_HIP_ERR_ARGUMENT, __func__, "batch too large");
  g_batch = n_images ? n_images : 1;
}
unsigned pulp_nn_hip_get_batch(void) { return g_batch; }
void pulp_nn_hip_set_stream(void *hip_stream) { g_stream = (hipStream_t)hip_stream; }
void *pulp_nn_hip_get_stream(void) { return (void *)g_stream; }

int pulp_nn_hip_sync(void)
{
  hipError_t e = hipStreamSynchronize(g_stream);
  if (e != hipSuccess) {
    set_error(PULP_NN_HIP_ERR_RUNTIME, __func__, hipGetErrorString(e));
    return PULP_NN_HIP_ERR_RUNTIME;
  }
  return PULP_NN_HIP_OK;
}

void pulp_nn_hip_clock_probe(long long *out)
{
  REQUIRE(out && aligned(out, 8), PULP_NN_HIP_ERR_ARGUMENT, "null or misaligned pointer");
  hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, g_stream, out);
  check_launch(__func__);
}

int pulp_nn_hip_last_error(void) { return g_err; }
const char *pulp_nn_hip_last_error_string(void) { return g_errmsg; }
void pulp_nn_hip_clear_error(void)
{
  g_err = PULP_NN_HIP_OK;
  g_errmsg[0] = 0;
}
int pulp_nn_hip_bn_bits(void) { return PULPNN_BN_BITS; }

void pulp_nn_hip_hwc_to_chw(const unsigned char *in_hwc, unsigned char *out_chw, unsigned dim_x, unsigned dim_y,
                            unsigned ch, unsigned pad_top, unsigned pad_bottom)
{
  REQUIRE(in_hwc && out_chw, PULP_NN_HIP_ERR_ARGUMENT, "null pointer");
  REQUIRE(dim_x && dim_y && ch, PULP_NN_HIP_ERR_ARGUMENT, "zero dimension");
  const unsigned hw = dim_x * dim_y, plane = (pad_top + dim_y + pad_bottom) * dim_x;
  if (ch % 16 == 0 && hw % 4 == 0 && plane % 4 == 0 && (pad_top * dim_x) % 4 == 0 && aligned(in_hwc, 16) &&
      aligned(out_chw, 4)) {
    const int tiles_p = (int)((hw + 255) / 256), tiles_c = (int)((ch + 63) / 64);
    const long long total = (long long)g_batch * tiles_p * tiles_c;
    REQUIRE(total <= 0x7fffffffLL, PULP_NN_HIP_ERR_ARGUMENT, "batch too large");
    if ((long long)g_batch * hw * ch >= PULPNN_NT_BYTES)
      hipLaunchKernelGGL(hwc_to_chw_fast_kernel<true>, dim3((unsigned)total), dim3(256), 0, g_stream, in_hwc, out_chw,
                         (int)dim_y, (int)dim_x, (int)ch, (int)pad_top, (int)pad_bottom, tiles_p, tiles_c);
    else
      hipLaunchKernelGGL(hwc_to_chw_fast_kernel<false>, dim3((unsigned)total), dim3(256), 0, g_stream, in_hwc, out_chw,
                         (int)dim_y, (int)dim_x, (int)ch, (int)pad_top, (int)pad_bottom, tiles_p, tiles_c);
    check_launch(__func__);
    return;
  }
  const int tiles_p = (int)((dim_x * dim_y + 63) / 64), tiles_c = (int)((ch + 63) / 64);
  const long long total = (long long)g_batch * tiles_p * tiles_c;
  REQUIRE(total <= 0x7fffffffLL, PULP_NN_HIP_ERR_ARGUMENT, "batch too large");
  hipLaunchKernelGGL(hwc_to_chw_kernel, dim3((unsigned)total), dim3(256), 0, g_stream, in_hwc, out_chw, (int)dim_y,
                     (int)dim_x, (int)ch, (int)pad_top, (int)pad_bottom, tiles_p, tiles_c);
  check_launch(__func__);
}

unsigned long long pulp_nn_hip_calib_workspace_bytes(unsigned long long n_outputs)
{
  return ((n_outputs + CALIB_CHUNK - 1) / CALIB_CHUNK) * sizeof(unsigned long long);
}

void pulp_nn_hip_calib_conv(const unsigned char *pInBuffer, const signed char *bias, const signed char *pWeight,
                            const void *k, unsigned short dim_in_x, unsigned short dim_in_y, unsigned short ch_in,
                            unsigned short dim_out_x, unsigned short dim_out_y, unsigned short ch_out,
                            unsigned short dim_kernel_x, unsigned short dim_kernel_y, unsigned short padding_y_top,
                            unsigned short padding_x_left, unsigned short stride_x, unsigned short stride_y,
                            void *workspace, unsigned long long workspace_bytes, unsigned long long *result)
{
  CalibGeom g = calib_conv_geom(pInBuffer, bias, pWeight, k, dim_in_x, dim_in_y, ch_in, dim_out_x, dim_out_y, ch_out,
                                dim_kernel_x, dim_kernel_y, padding_y_top, padding_x_left, stride_x, stride_y);
  REQUIRE(aligned(workspace, 8) && aligned(result, 8), PULP_NN_HIP_ERR_ARGUMENT, "workspace and result must be 8-byte aligned");
  calib_common(__func__, g, (unsigned long long *)workspace, workspace_bytes / sizeof(unsigned long long), result);
}

void pulp_nn_hip_calib_conv_static(const unsigned char *pInBuffer, const signed char *bias, const signed char *pWeight,
                                   const void *k, unsigned short dim_in_x, unsigned short dim_in_y,
                                   unsigned short ch_in, unsigned short dim_out_x, unsigned short dim_out_y,
                                   unsigned short ch_out, unsigned short dim_kernel_x, unsigned short dim_kernel_y,
                                   unsigned short padding_y_top, unsigned short padding_x_left,
                                   unsigned short stride_x, unsigned short stride_y, unsigned long long *result)
{
  CalibGeom g = calib_conv_geom(pInBuffer, bias, pWeight, k, dim_in_x, dim_in_y, ch_in, dim_out_x, dim_out_y, ch_out,
                                dim_kernel_x, dim_kernel_y, padding_y_top, padding_x_left, stride_x, stride_y);
  REQUIRE(aligned(result, 8), PULP_NN_HIP_ERR_ARGUMENT, "result must be 8-byte aligned");
  unsigned long long *partial = static_scratch(__func__);
  if (!partial) return;
  calib_common(__func__, g, partial, CALIB_STATIC_SLOTS, result);
}

void pulp_nn_hip_calib_depthwise(const unsigned char *Im_in, const signed char *bias, const signed char *wt,
                                 const void *k, unsigned short dim_im_in_x, unsigned short dim_im_in_y,
                                 unsigned short ch, unsigned short dim_im_out_x, unsigned short dim_im_out_y,
                                 unsigned short dim_kernel_x, unsigned short dim_kernel_y, unsigned short padding_y_top,
                                 unsigned short padding_x_left, unsigned short stride_x, unsigned short stride_y,
                                 int input_is_hwc, void *workspace, unsigned long long workspace_bytes,
                                 unsigned long long *result)
{
  CalibGeom g = calib_conv_geom(Im_in, bias, wt, k, dim_im_in_x, dim_im_in_y, ch, dim_im_out_x, dim_im_out_y, ch,
                                dim_kernel_x, dim_kernel_y, padding_y_top, padding_x_left, stride_x, stride_y);
  g.depthwise = 1;
  g.chw_in = !input_is_hwc;
  REQUIRE(aligned(workspace, 8) && aligned(result, 8), PULP_NN_HIP_ERR_ARGUMENT, "workspace and result must be 8-byte aligned");
  calib_common(__func__, g, (unsigned long long *)workspace, workspace_bytes / sizeof(unsigned long long), result);
}

// ---- the reference API ------------------------------------------------------------

#define CONV_FORWARD(NAME, POINTWISE)                                                                   \
  void NAME(PULP_NN_CONV_ARGS)                                                                          \
  {                                                                                                     \
    (void)pIm2ColBuffer;                                                                                \
    (void)padding_y_bottom;                                                                             \
    (void)padding_x_right;                                                                              \
    conv_common(#NAME, POINTWISE, pInBuffer, bias, pOutBuffer, pWeight, k, lambda, out_mult, out_shift, \
                dim_in_x, dim_in_y, ch_in, dim_out_x, dim_out_y, ch_out, dim_kernel_x, dim_kernel_y,    \
                padding_y_top, padding_x_left, stride_x, stride_y, flag_relu, flag_batch_norm);         \
  }

CONV_FORWARD(pulp_nn_conv_Ho_parallel, false)
CONV_FORWARD(pulp_nn_conv_Co_parallel, false)
CONV_FORWARD(pulp_nn_conv_HoWo_parallel, false)
CONV_FORWARD(pulp_nn_pointwise_HoWo_parallel, true)
CONV_FORWARD(pulp_nn_pointwise_Ho_parallel, true)
CONV_FORWARD(pulp_nn_pointwise_Co_parallel, true)

void pulp_nn_linear(uint8_t *pInBuffer, int8_t *bias, uint8_t *pOutBuffer, int8_t *pWeights, bn_t *k, bn_t *lambda,
                    uint16_t out_mult, int8_t out_shift, uint16_t dim_vec, uint16_t num_o_neurons, int flag_relu,
                    int flag_batch_norm)
{
  const int mode = epi_mode(flag_relu, flag_batch_norm);
  EpiArgs e;
  REQUIRE(epi_args(mode, k, lambda, out_mult, out_shift, &e), PULP_NN_HIP_ERR_ARGUMENT,
          "out_shift out of range or null k/lambda");
  linear_common(__func__, mode, pInBuffer, bias, pOutBuffer, pWeights, e, dim_vec, num_o_neurons, (int)g_batch);
}

void pulp_nn_linear_out_32(uint8_t *pInBuffer, int8_t *bias, int32_t *pOutBuffer, int8_t *pWeights, uint16_t dim_vec,
                           uint16_t num_o_neurons)
{
  REQUIRE(!bias || aligned(bias, 4), PULP_NN_HIP_ERR_ARGUMENT, "bias must be 4-byte aligned (it holds int32 values)");
  REQUIRE(aligned(pOutBuffer, 4), PULP_NN_HIP_ERR_ARGUMENT, "output must be 4-byte aligned");
  EpiArgs e = {nullptr, nullptr, 0, 0};
  linear_common(__func__, EPI_OUT32, pInBuffer, bias, pOutBuffer, pWeights, e, dim_vec, num_o_neurons, (int)g_batch);
}

uint8_t *pulp_nn_matmul(const int8_t *pWeight, uint8_t *pInBuffer, uint16_t ch_out, uint16_t num_col_im2col,
                        uint16_t out_shift, uint16_t out_mult, bn_t *k, bn_t *lambda, const int8_t *bias, uint8_t *pOut,
                        uint8_t *pOut2, int flag_relu, int flag_batch_norm)
{
  const int mode = epi_mode(flag_relu, flag_batch_norm);
  EpiArgs e;
  if (!epi_args(mode, k, lambda, out_mult, out_shift, &e)) {
    set_error(PULP_NN_HIP_ERR_ARGUMENT, __func__, "out_shift out of range or null k/lambda");
    return pOut;
  }
  if (!pOut || !pOut2) {
    set_error(PULP_NN_HIP_ERR_ARGUMENT, __func__, "null pointer");
    return pOut;
  }
  if (pOut2 == pOut + ch_out) {
    linear_common(__func__, mode, pInBuffer, bias, pOut, pWeight, e, num_col_im2col, ch_out, 2);
  } else {
    linear_common(__func__, mode, pInBuffer, bias, pOut, pWeight, e, num_col_im2col, ch_out, 1);
    linear_common(__func__, mode, pInBuffer + num_col_im2col, bias, pOut2, pWeight, e, num_col_im2col, ch_out, 1);
  }
  return pOut + 2 * (size_t)ch_out;
}

void pulp_nn_maxpool(uint8_t *Im_in, uint8_t *Im_out, uint16_t dim_im_in_x, uint16_t dim_im_in_y, uint16_t ch_im_in,
                     uint16_t dim_im_out_x, uint16_t dim_im_out_y, uint16_t dim_kernel_x, uint16_t dim_kernel_y,
                     uint16_t padding_t, uint16_t padding_b, uint16_t padding_l, uint16_t padding_r, uint16_t stride_x,
                     uint16_t stride_y)
{
  PoolGeom g;
  if (!pool_geom(__func__, &g, Im_in, Im_out, dim_im_in_x, dim_im_in_y, ch_im_in, dim_im_out_x, dim_im_out_y,
                 dim_kernel_x, dim_kernel_y, padding_t, padding_b, padding_l, padding_r, stride_x, stride_y))
    return;
  // The reference's in-place x pass re-reads columns it has already overwritten
  // when a window starts left of the column it is stored to, i.e. for some
  // i_x >= 1 with i_x*stride_x - padding_l < i_x (pulp_nn_maxpool.c:58-94).
  REQUIRE(padding_l == 0 || (int)stride_x - 1 >= (int)padding_l, PULP_NN_HIP_ERR_UNSUPPORTED,
          "left padding this large makes the reference's in-place x pass order dependent");
  if (ch_im_in % 16 == 0 && aligned(Im_in, 16) && aligned(Im_out, 16)) {
    g.cgroups = ch_im_in / 16;
    g.total = (long long)g.B * g.Ho * g.Wo * g.cgroups;
    const dim3 grid((unsigned)((g.total + 255) / 256));
    // non-temporal loads: windows that do not overlap, on an input too large to find again in a cache
    const bool lnt = stride_x >= dim_kernel_x && stride_y >= dim_kernel_y &&
                     (long long)g.B * g.H * g.W * g.C >= PULPNN_NT_BYTES;
    const bool snt = g.total * 16 >= PULPNN_NT_BYTES;
    if (snt && lnt) hipLaunchKernelGGL((maxpool16_kernel<true, true>), grid, dim3(256), 0, g_stream, g);
    else if (snt) hipLaunchKernelGGL((maxpool16_kernel<true, false>), grid, dim3(256), 0, g_stream, g);
    else if (lnt) hipLaunchKernelGGL((maxpool16_kernel<false, true>), grid, dim3(256), 0, g_stream, g);
    else hipLaunchKernelGGL((maxpool16_kernel<false, false>), grid, dim3(256), 0, g_stream, g);
  } else {
    hipLaunchKernelGGL(maxpool_kernel, dim3((unsigned)((g.total + 255) / 256)), dim3(256), 0, g_stream, g);
  }
  check_launch(__func__);
}

void pulp_nn_avgpool(uint8_t *Im_in, uint8_t *Im_out, bn_t lambda, uint16_t out_shift, bn_t out_add,
                     uint16_t dim_im_in_x, uint16_t dim_im_in_y, uint16_t ch_im_in, uint16_t dim_im_out_x,
                     uint16_t dim_im_out_y, uint16_t dim_kernel_x, uint16_t dim_kernel_y, uint16_t padding_t,
                     uint16_t padding_b, uint16_t padding_l, uint16_t padding_r, uint16_t stride_x, uint16_t stride_y,
                     int flag_requant)
{
  PoolGeom g;
  if (!pool_geom(__func__, &g, Im_in, Im_out, dim_im_in_x, dim_im_in_y, ch_im_in, dim_im_out_x, dim_im_out_y,
                 dim_kernel_x, dim_kernel_y, padding_t, padding_b, padding_l, padding_r, stride_x, stride_y))
    return;
  REQUIRE(!flag_requant || out_shift < PULPNN_BN_BITS, PULP_NN_HIP_ERR_ARGUMENT, "out_shift out of range");
  REQUIRE((long long)dim_kernel_x * dim_kernel_y * 255 < 0xffffffffLL, PULP_NN_HIP_ERR_UNSUPPORTED, "window too large");
  AvgArgs a = {(long long)lambda, (long long)out_add, (int)out_shift, flag_requant};
  hipLaunchKernelGGL(avgpool_kernel, dim3((unsigned)((g.total + 255) / 256)), dim3(256), 0, g_stream, g, a);
  check_launch(__func__);
}

void pulp_nn_add(uint8_t *Im_in_1, uint8_t *Im_in_2, uint8_t *Im_out, uint16_t out_mult1, uint16_t out_mult2,
                 uint16_t out_shift, uint16_t dim_im_in_h, uint16_t dim_im_in_w, uint16_t ch_im_in)
{
  REQUIRE(Im_in_1 && Im_in_2 && Im_out, PULP_NN_HIP_ERR_ARGUMENT, "null pointer");
  REQUIRE(dim_im_in_h && dim_im_in_w && ch_im_in, PULP_NN_HIP_ERR_ARGUMENT, "zero dimension");
  const int d = (int)(int8_t)out_shift;  // pulp_nn_add_quant_u8 takes the shift as int8_t
  REQUIRE(d >= 0 && d < 32, PULP_NN_HIP_ERR_ARGUMENT, "out_shift out of range");
  const long long n = (long long)g_batch * dim_im_in_h * dim_im_in_w * ch_im_in;
  const long long threads = (n + 15) / 16;
  REQUIRE((threads + 255) / 256 <= 0x7fffffffLL, PULP_NN_HIP_ERR_ARGUMENT, "batch too large");
  const int vec16 = aligned(Im_in_1, 16) && aligned(Im_in_2, 16) && aligned(Im_out, 16);
  hipLaunchKernelGGL(add_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, g_stream, Im_in_1, Im_in_2,
                     Im_out, n, (int)(int16_t)out_mult1, (int)(int16_t)out_mult2, d, vec16);
  check_launch(__func__);
}

#define DW_FORWARD(NAME)                                                                                       \
  void NAME(PULP_NN_DW_ARGS)                                                                                   \
  {                                                                                                            \
    (void)bufferC;                                                                                             \
    (void)bufferB;                                                                                             \
    (void)ch_im_in;                                                                                            \
    (void)padding_y_bottom;                                                                                    \
    (void)padding_x_right;                                                                                     \
    depthwise_common(#NAME, Im_in, bias, Im_out, wt, k, lambda, out_mult, out_shift, dim_im_in_x, dim_im_in_y, \
                     dim_im_out_x, dim_im_out_y, ch_im_out, dim_kernel_x, dim_kernel_y, padding_y_top,         \
                     padding_x_left, stride_x, stride_y, epi_mode(FLAG_RELU, FLAG_BATCH_NORM, true));          \
  }

DW_FORWARD(pulp_nn_depthwise_generic)
DW_FORWARD(pulp_nn_depthwise_generic_less_4_weights)

void pulp_nn_hip_depthwise_hwc(const unsigned char *Im_in, const signed char *bias, unsigned char *Im_out,
                               const signed char *wt, void *k, void *lambda, unsigned short out_mult,
                               unsigned short out_shift, unsigned short dim_im_in_x, unsigned short dim_im_in_y,
                               unsigned short ch, unsigned short dim_im_out_x, unsigned short dim_im_out_y,
                               unsigned short stride, signed char flag_relu, signed char flag_batch_norm)
{
  depthwise_common(__func__, Im_in, (const int8_t *)bias, Im_out, (const int8_t *)wt, (bn_t *)k, (bn_t *)lambda, out_mult,
                   out_shift, dim_im_in_x, dim_im_in_y, dim_im_out_x, dim_im_out_y, ch, 3, 3, 1, 1, stride, stride,
                   epi_mode(flag_relu, flag_batch_norm, true), true);
}

// Common part of pulp_nn_hip_dw_pw_hwc (one block) and pulp_nn_hip_dw_pw_chain_hwc (several).
static void dwpw_common(const char *fn, const unsigned char *Im_in, unsigned char *Im_out, int W, int H, int C, int Wo_arg,
                        int Ho_arg, int Co, int S, unsigned n_blocks, const pulp_nn_hip_block *blocks)
{
  REQUIRE(Im_in && Im_out && blocks && n_blocks >= 1, PULP_NN_HIP_ERR_ARGUMENT, "null activation pointer or no block");
  REQUIRE(n_blocks <= DWPW_MAX_BLOCKS, PULP_NN_HIP_ERR_ARGUMENT, "too many blocks for one launch");
  REQUIRE(W && H && C && Co && (S == 1 || S == 2), PULP_NN_HIP_ERR_ARGUMENT, "zero dimension or stride other than 1 or 2");
  const int Wo = (W - 1) / S + 1, Ho = (H - 1) / S + 1;
  REQUIRE(Wo_arg == Wo && Ho_arg == Ho, PULP_NN_HIP_ERR_ARGUMENT, "output size is not that of a 3x3 window with padding 1");
  DwPwGeom g;
  g.nblocks = (int)n_blocks;
  bool w_aligned = true;
  for (unsigned j = 0; j < n_blocks; j++) {
    const pulp_nn_hip_block &b = blocks[j];
    REQUIRE(b.dw_wt && b.pw_weight, PULP_NN_HIP_ERR_ARGUMENT, "null weight pointer");
    DwPwBlock &P = g.blk[j];
    P.dw_wt = (const int8_t *)b.dw_wt;
    P.dw_bias = (const int8_t *)b.dw_bias;
    P.pw_w = (const int8_t *)b.pw_weight;
    P.pw_bias = (const int8_t *)b.pw_bias;
    P.mode_dw = epi_mode(b.dw_flag_relu, b.dw_flag_batch_norm, true);  // pulp_nn_depthwise_generic.c:167-178 tests FLAG_RELU for truth
    P.mode_pw = epi_mode(b.pw_flag_relu, b.pw_flag_batch_norm);
    REQUIRE(epi_args(P.mode_dw, (bn_t *)b.dw_k, (bn_t *)b.dw_lambda, b.dw_out_mult, b.dw_out_shift, &P.e_dw) &&
                epi_args(P.mode_pw, (bn_t *)b.pw_k, (bn_t *)b.pw_lambda, b.pw_out_mult, b.pw_out_shift, &P.e_pw),
            PULP_NN_HIP_ERR_ARGUMENT, "out_shift out of range or null k/lambda");
    w_aligned = w_aligned && aligned(b.pw_weight, 16);
  }
  // per input width and stride: output rows of a stage-1 item, waves per workgroup, pixels / 16 of a stage-2 block
  int R = 0, NWV = 4, TMB = 2;
  if (W == 64) R = 2;
  else if (W == 32) R = 4;
  else if (W == 16) { R = S == 1 ? 4 : 2; NWV = 8; TMB = 2; }
  else if (W == 8) { R = S == 1 ? 4 : 2; NWV = 8; TMB = 2; }
  else if (W == 4 && S == 1) { R = 4; NWV = 8; TMB = 2; }
  const bool c_ok = (C == 16 || C == 32 || (C % 64 == 0 && C <= 1024));
  const int LG = C >= 64 ? 1 : 64 / C, CGN = C >= 64 ? C / 64 : 1;
  const long long M = (long long)g_batch * Ho * Wo;
  const bool ok = R > 0 && c_ok && Ho % (R * LG) == 0 && Co % 16 == 0 && aligned(Im_in, 4) && aligned(Im_out, 16) &&
                  w_aligned && M <= 0x7fffffffLL && (long long)Co * C < 0x7fffffffLL;
  if (!ok)
    return set_error(PULP_NN_HIP_ERR_UNSUPPORTED, fn, "no fused kernel for this geometry: call the depthwise and the pointwise layer separately");
  g.in = Im_in;
  g.out = Im_out;
  g.B = (int)g_batch;
  g.C = C;
  g.H = H;
  g.Ho = Ho;
  g.Co = Co;
  g.M = (int)M;
  g.KT = (C + 63) / 64;
  g.d_howo = fastdiv_make((unsigned)(Ho * Wo));
  // a tile: enough stage-1 items (item_px pixels x 64 channels each) to give every wave one, in whole stage-2 blocks
  const int item_px = R * LG * Wo, bp = 16 * TMB;
  int segs = (NWV + CGN - 1) / CGN;                       // items along the pixels
  while ((segs * item_px) % bp) segs++;
  while (segs > 1 && (dwpw_lds_bytes(segs * item_px, C) > 49152 || (M + (long long)segs * item_px - 1) / (segs * item_px) < num_cus()))
    segs--;
  while ((segs * item_px) % bp) segs++;
  g.BM = segs * item_px;
  int tiles = (int)((M + g.BM - 1) / g.BM);
  const int nbt = (Co + 63) / 64;
  // few pixel tiles: several workgroups share one, each with a part of the output channels (and its own copy of stage 1)
  g.nsplit = 1;
  while (tiles * g.nsplit < num_cus() && g.nsplit * 2 <= nbt) g.nsplit *= 2;
  // (the kernel stages the pointwise constants of at most 1024 channels per workgroup)
  if (((nbt + g.nsplit - 1) / g.nsplit) * 64 > 1024)
    return set_error(PULP_NN_HIP_ERR_UNSUPPORTED, fn, "more than 1024 output channels per workgroup: call the depthwise and the pointwise layer separately");
  size_t lds = (size_t)dwpw_lds_bytes(g.BM, C) + (size_t)dwpw_const_bytes(((nbt + g.nsplit - 1) / g.nsplit) * 64);
  if (n_blocks > 1) {
    // Several blocks: the output of one is the next one's input and stays in LDS, so a tile has to be whole images
    // (the 3x3 window of a pixel then never leaves the tile), the blocks have to keep the shape (stride 1, as many
    // channels out as in), and a workgroup computes all channels.
    const int img_px = Ho * Wo;
    int per_tile = (g.BM + img_px - 1) / img_px;  // images per tile
    while ((per_tile * img_px) % bp || (per_tile * img_px) % item_px) per_tile++;
    g.BM = per_tile * img_px;
    tiles = (int)((M + g.BM - 1) / g.BM);
    g.nsplit = 1;
    lds = (size_t)dwpw_lds_bytes(g.BM, C) + (size_t)dwpw_const_bytes(nbt * 64) + (size_t)g.BM * (Co + DWPW_YPAD);
    if (S != 1 || C != Co || g_batch % (unsigned)per_tile != 0)
      return set_error(PULP_NN_HIP_ERR_UNSUPPORTED, fn, "blocks can only be chained at stride 1 with as many channels out as in, on whole images per tile");
  }
  if (lds > 65536)
    return set_error(PULP_NN_HIP_ERR_UNSUPPORTED, fn, "no fused kernel for this geometry: call the depthwise and the pointwise layer separately");
  const dim3 grid((unsigned)(tiles * g.nsplit)), block(64 * NWV);
#define DWPW_KP(WB, RR, SS, NW, TM)                                                                    \
  if (g.KT == 1) hipLaunchKernelGGL((dwpw_fused_kernel<WB, RR, SS, NW, TM, 1>), grid, block, lds, g_stream, g);      \
  else if (g.KT == 2) hipLaunchKernelGGL((dwpw_fused_kernel<WB, RR, SS, NW, TM, 2>), grid, block, lds, g_stream, g); \
  else hipLaunchKernelGGL((dwpw_fused_kernel<WB, RR, SS, NW, TM, 4>), grid, block, lds, g_stream, g);
#define DWPW_CHAIN_KP(WB, RR, NW, TM)                                                                                     \
  if (g.KT == 1) hipLaunchKernelGGL((dwpw_fused_kernel<WB, RR, 1, NW, TM, 1, true>), grid, block, lds, g_stream, g);      \
  else if (g.KT == 2) hipLaunchKernelGGL((dwpw_fused_kernel<WB, RR, 1, NW, TM, 2, true>), grid, block, lds, g_stream, g); \
  else hipLaunchKernelGGL((dwpw_fused_kernel<WB, RR, 1, NW, TM, 4, true>), grid, block, lds, g_stream, g);
  if (n_blocks > 1) {
    // (stride 1 only; the widest planes never fit the LDS of a chained launch)
    if (W == 32) { DWPW_CHAIN_KP(32, 4, 4, 2) }
    else if (W == 16) { DWPW_CHAIN_KP(16, 4, 8, 2) }
    else if (W == 8) { DWPW_CHAIN_KP(8, 4, 8, 2) }
    else if (W == 4) { DWPW_CHAIN_KP(4, 4, 8, 2) }
    else return set_error(PULP_NN_HIP_ERR_UNSUPPORTED, fn, "blocks of this width cannot be chained");
    check_launch(fn);
    return;
  }
  if (W == 64 && S == 1) { DWPW_KP(64, 2, 1, 4, 2) }
  else if (W == 64) { DWPW_KP(64, 2, 2, 4, 2) }
  else if (W == 32 && S == 1) { DWPW_KP(32, 4, 1, 4, 2) }
  else if (W == 32) { DWPW_KP(32, 4, 2, 4, 2) }
  else if (W == 16 && S == 1) { DWPW_KP(16, 4, 1, 8, 2) }
  else if (W == 16) { DWPW_KP(16, 2, 2, 8, 2) }
  else if (W == 8 && S == 1) { DWPW_KP(8, 4, 1, 8, 2) }
  else if (W == 8) { DWPW_KP(8, 2, 2, 8, 2) }
  else { DWPW_KP(4, 4, 1, 8, 2) }
#undef DWPW_KP
#undef DWPW_CHAIN_KP
  check_launch(fn);
}

void pulp_nn_hip_dw_pw_hwc(const unsigned char *Im_in, unsigned char *Im_out, unsigned short dim_im_in_x,
                           unsigned short dim_im_in_y, unsigned short ch, unsigned short dim_im_out_x,
                           unsigned short dim_im_out_y, unsigned short ch_out, unsigned short stride,
                           const signed char *dw_wt, const signed char *dw_bias, void *dw_k, void *dw_lambda,
                           unsigned short dw_out_mult, unsigned short dw_out_shift, signed char dw_flag_relu,
                           signed char dw_flag_batch_norm, const signed char *pw_weight, const signed char *pw_bias,
                           void *pw_k, void *pw_lambda, unsigned short pw_out_mult, unsigned short pw_out_shift,
                           signed char pw_flag_relu, signed char pw_flag_batch_norm)
{
  const pulp_nn_hip_block b = {dw_wt,     dw_bias,   dw_k,        dw_lambda,    dw_out_mult,  dw_out_shift, dw_flag_relu, dw_flag_batch_norm,
                               pw_weight, pw_bias,   pw_k,        pw_lambda,    pw_out_mult,  pw_out_shift, pw_flag_relu, pw_flag_batch_norm};
  dwpw_common(__func__, Im_in, Im_out, dim_im_in_x, dim_im_in_y, ch, dim_im_out_x, dim_im_out_y, ch_out, stride, 1, &b);
}

void pulp_nn_hip_dw_pw_chain_hwc(const unsigned char *Im_in, unsigned char *Im_out, unsigned short dim_im_x,
                                 unsigned short dim_im_y, unsigned short ch, unsigned n_blocks,
                                 const pulp_nn_hip_block *blocks)
{
  dwpw_common(__func__, Im_in, Im_out, dim_im_x, dim_im_y, ch, dim_im_x, dim_im_y, ch, 1, n_blocks, blocks);
}

void pulp_nn_depthwise_3x3_s1(uint8_t *In_Img, uint8_t *Out_Img, int R, int C, int CH, int p_l, int p_r,
                              int8_t *Kernel, int8_t out_shift, uint16_t out_mult, bn_t *kappa, bn_t *lambda,
                              int flag_relu, int flag_batch_norm, unsigned int *memory_chan)
{
  (void)memory_chan;
  REQUIRE(R >= 3 && C >= 2 && CH >= 1, PULP_NN_HIP_ERR_ARGUMENT, "plane too small");
  REQUIRE(R <= 65535 + 2 && C <= 65535 && CH <= 65535, PULP_NN_HIP_ERR_ARGUMENT, "dimension too large");
  // Only for p_l = p_r = 1 and even C do the reference's three row pointers land on
  // the start of the next row after each output row (pulp_nn_depthwise_3x3_s1.c:141-223).
  REQUIRE(p_l == 1 && p_r == 1 && (C % 2) == 0, PULP_NN_HIP_ERR_UNSUPPORTED,
          "only p_l = p_r = 1 with even C is well defined in the reference");
  depthwise_common(__func__, In_Img, nullptr, Out_Img, Kernel, kappa, lambda, out_mult, out_shift, C, R, C, R - 2, CH,
                   3, 3, 0, 1, 1, 1, epi_mode(flag_relu, flag_batch_norm));
}

}  // extern "C"
