// Direct convolution for layers whose whole filter is at most 32 bytes long
// (K = ky * kx * Ci <= 32) and that have at most 32 output channels: the stem of
// a network (3x3 on RGB, 27 bytes per output channel).
//
// Such a layer is pure streaming (a few hundred multiply-adds per pixel against
// tens of bytes moved) and a GEMM tile is mostly padding for it, so it is done
// with v_dot4 on the vector ALUs instead: one output pixel per lane, its K input
// bytes gathered into 8 dwords (bytes past K and taps outside the image as zero),
// all weights and per-channel constants broadcast from LDS, the NCH results of a
// pixel packed and written as 16-byte pieces, one contiguous run per wave.
//
// Arithmetic as in igemm.h: activations as a ^ 0x80 with bias + 128 * sum_k w
// added back; exact in wrapping 32-bit arithmetic.
// Reference semantics: 32bit/src/pulp_nn_conv_Ho_parallel.c:76-183 (im2col order
// ky, kx, ci) and pulp_nn_matmul.c:144-216 (requantisation).
#pragma once
#include <type_traits>

#include "igemm.h"
#include "memops.h"
#include "requant.h"

#define SMALLK_KD 8  // filter dwords per channel (K <= 32)

template <int NCH, int MODE>
__global__ __launch_bounds__(256) void smallk_conv_kernel(ConvGeom g, EpiArgs e)
{
  __shared__ __attribute__((aligned(16))) int wl[NCH * SMALLK_KD];  // [channel][dword]
  __shared__ int corr_l[NCH];
  __shared__ bn_t k_l[NCH], lam_l[NCH];

  const int tid = threadIdx.x;
  // ---- weights and constants -> LDS -------------------------------------------------
  for (int q = tid; q < NCH * SMALLK_KD; q += 256) {
    const int n = q / SMALLK_KD, d = q % SMALLK_KD;
    unsigned v = 0;
    if (n < g.N) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int kk = 4 * d + j;
        if (kk < g.K) v |= (unsigned)(uint8_t)g.w[(long long)n * g.K + kk] << (8 * j);
      }
    }
    wl[q] = (int)v;
  }
  __syncthreads();
  if (tid < NCH) {
    int sum = 0;
#pragma unroll
    for (int d = 0; d < SMALLK_KD; d++) sum = __builtin_amdgcn_sdot4(wl[tid * SMALLK_KD + d], 0x01010101, sum, false);
    const bool real = tid < g.N;
    corr_l[tid] = 128 * sum + ((real && g.bias) ? (int)g.bias[tid] : 0);
    if (MODE == EPI_BN) {
      k_l[tid] = real ? e.k[tid] : 0;
      lam_l[tid] = real ? e.lambda[tid] : 0;
    }
  }
  __syncthreads();

  // ---- this lane's pixel: gather its K bytes -------------------------------------------
  const int m = blockIdx.x * 256 + tid;
  if (m >= g.M) return;
  const int b = m / g.HoWo, rem = m - b * g.HoWo;
  const int oy = rem / g.Wo, ox = rem - oy * g.Wo;
  const int iy0 = oy * g.sy - g.pt, ix0 = ox * g.sx - g.pl;
  const uint8_t *img = g.in + (long long)b * g.in_img;
  unsigned a[SMALLK_KD];
#pragma unroll
  for (int d = 0; d < SMALLK_KD; d++) a[d] = 0;
  {
    int fy = 0, fx = 0, ci = 0;
#pragma unroll
    for (int j = 0; j < 4 * SMALLK_KD; j++) {
      if (j < g.K) {
        const int iy = iy0 + fy, ix = ix0 + fx;
        if ((unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W)
          a[j >> 2] |= (unsigned)img[((long long)iy * g.W + ix) * g.Ci + ci] << (8 * (j & 3));
      }
      if (++ci == g.Ci) {
        ci = 0;
        if (++fx == g.kx) { fx = 0; ++fy; }
      }
    }
  }
#pragma unroll
  for (int d = 0; d < SMALLK_KD; d++) a[d] ^= 0x80808080u;

  // ---- NCH dot products, requantise, store ----------------------------------------------
  unsigned packed[NCH / 4];
#pragma unroll
  for (int n4 = 0; n4 < NCH / 4; n4++) {
    int acc[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int n = 4 * n4 + r;
      acc[r] = corr_l[n];
      const v4i w0 = *(const v4i *)&wl[n * SMALLK_KD], w1 = *(const v4i *)&wl[n * SMALLK_KD + 4];
      acc[r] = __builtin_amdgcn_sdot4((int)a[0], w0.x, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[1], w0.y, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[2], w0.z, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[3], w0.w, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[4], w1.x, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[5], w1.y, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[6], w1.z, acc[r], false);
      acc[r] = __builtin_amdgcn_sdot4((int)a[7], w1.w, acc[r], false);
    }
    unsigned p = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int n = 4 * n4 + r;
      const bn_t kk = (MODE == EPI_BN) ? k_l[n] : (bn_t)0, ll = (MODE == EPI_BN) ? lam_l[n] : (bn_t)0;
      p |= (unsigned)requant<MODE>(acc[r], kk, ll, e.mult, e.shift) << (8 * r);
    }
    packed[n4] = p;
  }
  uint8_t *o = (uint8_t *)g.out + (long long)m * g.N;
  if (g.vec_store) {
    // N == NCH and 16-byte aligned rows: one copy of the store code per cache policy
    auto put = [&](auto nt) {
      constexpr bool NT = decltype(nt)::value;
#pragma unroll
      for (int q = 0; q < NCH / 16; q++)
        store16<NT>(o + 16 * q, (v4i){(int)packed[4 * q], (int)packed[4 * q + 1], (int)packed[4 * q + 2], (int)packed[4 * q + 3]});
    };
    if (g.nt) put(std::true_type{});
    else put(std::false_type{});
  } else {
#pragma unroll
    for (int n = 0; n < NCH; n++)
      if (n < g.N) o[n] = (uint8_t)(packed[n >> 2] >> (8 * (n & 3)));
  }
}

// The same for filters of at most 3 rows whose rows (kx * Ci bytes, contiguous in the HWC
// input) are at most 9 bytes long, or at most 12 with Ci % 4 == 0: the 3x3 stem on RGB or
// RGBA.  A filter row of a pixel is fetched as one range-checked 12-byte buffer load from the
// aligned address below it (a row outside the image is an out-of-range load, which returns
// zeros) and shifted into place, instead of byte by byte: 3 loads per pixel instead of 27.  Filter rows are padded
// to 12 bytes in the weight table, so bytes past the end of a row meet zero weights; columns
// outside the image are masked to zero.
#define SMALLK_RD 3                  // dwords per filter row
#define SMALLK_RP (3 * SMALLK_RD + 3)  // weight table pitch per channel (12 dwords: 16-byte reads)

template <int NCH, int MODE>
__global__ __launch_bounds__(256) void smallk_rows_kernel(ConvGeom g, EpiArgs e)
{
  __shared__ __attribute__((aligned(16))) int wl[NCH * SMALLK_RP];  // [channel][row][dword]
  __shared__ int corr_l[NCH];
  __shared__ bn_t k_l[NCH], lam_l[NCH];
  __shared__ int k_small_l;

  const int tid = threadIdx.x;
  const int L = g.kx * g.Ci;  // bytes per filter row
  // ---- weights and constants -> LDS -------------------------------------------------
  for (int q = tid; q < NCH * SMALLK_RP; q += 256) {
    const int n = q / SMALLK_RP, d = q % SMALLK_RP, fy = d / SMALLK_RD, i = d % SMALLK_RD;
    unsigned v = 0;
    if (n < g.N && fy < g.ky) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int kk = 4 * i + j;
        if (kk < L) v |= (unsigned)(uint8_t)g.w[(long long)n * g.K + fy * L + kk] << (8 * j);
      }
    }
    wl[q] = (int)v;
  }
  __syncthreads();
  if (tid < NCH) {
    int sum = 0;
#pragma unroll
    for (int d = 0; d < 3 * SMALLK_RD; d++) sum = __builtin_amdgcn_sdot4(wl[tid * SMALLK_RP + d], 0x01010101, sum, false);
    const bool real = tid < g.N;
    corr_l[tid] = 128 * sum + ((real && g.bias) ? (int)g.bias[tid] : 0);
    bn_t kv = 0;
    if (MODE == EPI_BN) {
      kv = real ? e.k[tid] : 0;
      k_l[tid] = kv;
      lam_l[tid] = real ? e.lambda[tid] : 0;
    }
    // do all multipliers fit the fast form of the requantisation?  (NCH <= 64: these lanes are one wave)
    const bool all_small = __all(bn_k_small(kv));
    if (tid == 0) k_small_l = all_small;
  }
  __syncthreads();
  const bool k_small = k_small_l != 0;

  // ---- this lane's pixels: the (up to) three filter rows of each ---------------------------------
  // A workgroup takes g.tiles_n runs of 256 consecutive pixels (the weight table and the two barriers above are
  // set up once for all of them, not once per 256 pixels); the rows of the next run's pixel are requested before
  // this run's pixel is multiplied.
  const unsigned batch = (unsigned)((g.M + g.HoWo - 1) / g.HoWo);
  const int total = (int)(batch * (unsigned)g.in_img);  // bytes of input
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)g.in, 0, total, 0x00020000);
  typedef unsigned v3u __attribute__((ext_vector_type(3)));
  struct Rows {
    v3u d[3];              // the 12 bytes from the aligned address below each row's first byte
    int sh[3];             // where the row starts in them
    unsigned md[SMALLK_RD];  // byte mask of the columns inside the image
    int A0, lo, hi, iy0;   // (for the few lanes whose load would leave the input: see finish())
    bool ok[3];
  };
  auto request = [&](int m, Rows &R) {
    const bool live = m < g.M;
    const int mm = live ? m : 0;
    const int b = (int)fastdiv((unsigned)mm, g.d_howo), rem = mm - b * g.HoWo;
    const int oy = (int)fastdiv((unsigned)rem, g.d_wo), ox = rem - oy * g.Wo;
    const int iy0 = oy * g.sy - g.pt, ix0 = ox * g.sx - g.pl;
    // bytes [lo, hi) of a filter row lie inside the image
    const int lo = max(0, -ix0) * g.Ci, hi = max(min(g.kx, g.W - ix0), 0) * g.Ci;
    const unsigned bits = ((1u << hi) - 1u) & ~((1u << lo) - 1u);  // hi <= 12
#pragma unroll
    for (int i = 0; i < SMALLK_RD; i++) R.md[i] = ((((bits >> (4 * i)) & 15u) * 0x00204081u) & 0x01010101u) * 0xFFu;
    const int rowpos = (int)((unsigned)b * (unsigned)g.in_img) + ix0 * g.Ci;  // byte offset of the row's first byte, less iy * W * Ci
    R.A0 = rowpos, R.lo = lo, R.hi = hi, R.iy0 = iy0;
#pragma unroll
    for (int fy = 0; fy < 3; fy++) {
      const int iy = iy0 + fy;
      R.ok[fy] = live && fy < g.ky && (unsigned)iy < (unsigned)g.H;
      const int A = rowpos + iy * g.W * g.Ci;
      R.sh[fy] = A & 3;
      // one range-checked load; a row outside the image is given an offset that is out of range, which loads zeros
      R.d[fy] = __builtin_amdgcn_raw_buffer_load_b96(rsrc, R.ok[fy] ? A - R.sh[fy] : (int)0xfffffff0, 0, 0);
    }
  };
  auto finish = [&](const Rows &R, unsigned (&a)[3][SMALLK_RD]) {
#pragma unroll
    for (int fy = 0; fy < 3; fy++) {
      unsigned r0 = __builtin_amdgcn_alignbyte(R.d[fy].y, R.d[fy].x, R.sh[fy]);
      unsigned r1 = __builtin_amdgcn_alignbyte(R.d[fy].z, R.d[fy].y, R.sh[fy]);
      unsigned r2 = __builtin_amdgcn_alignbyte(0u, R.d[fy].z, R.sh[fy]);
      // The load must lie inside the input as a whole.  Where it would not (left padding in the
      // first row of the first image, the last bytes of the last image), the few lanes concerned
      // fetch the bytes of the row that lie inside the image one by one.
      const int A = R.A0 + (R.iy0 + fy) * g.W * g.Ci, base = A - R.sh[fy];
      if (R.ok[fy] && (base < 0 || base + 12 > total)) {
        unsigned t[SMALLK_RD] = {0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4 * SMALLK_RD; j++)
          if (j >= R.lo && j < R.hi) t[j >> 2] |= (unsigned)g.in[A + j] << (8 * (j & 3));
        r0 = t[0];
        r1 = t[1];
        r2 = t[2];
      }
      a[fy][0] = (r0 & R.md[0]) ^ 0x80808080u;
      a[fy][1] = (r1 & R.md[1]) ^ 0x80808080u;
      a[fy][2] = (r2 & R.md[2]) ^ 0x80808080u;
    }
  };
  const int npass = g.tiles_n;
  int m = blockIdx.x * npass * 256 + tid;
  Rows cur, nxt;
  request(m, cur);
#pragma unroll 1
  for (int pass = 0; pass < npass; pass++, m += 256) {
    if (pass + 1 < npass) request(m + 256, nxt);
    unsigned a[3][SMALLK_RD];
    finish(cur, a);

    // ---- NCH dot products, requantise, store ----------------------------------------------
    // (the weight table is read through an offset the compiler cannot see through: known to be the same in every
    // pass, all NCH x 9 weight dwords would be read before the loop and kept in registers, 2 waves per SIMD fit then)
    int wofs = 0;
    asm volatile("" : "+s"(wofs));
    const int *wt = wl + wofs;
    unsigned packed[NCH / 4];
#pragma unroll
    for (int n4 = 0; n4 < NCH / 4; n4++) {
      int acc[4];
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int n = 4 * n4 + r;
        acc[r] = corr_l[n];
        const v4i w0 = *(const v4i *)&wt[n * SMALLK_RP], w1 = *(const v4i *)&wt[n * SMALLK_RP + 4];
        const int w2 = wt[n * SMALLK_RP + 8];
        acc[r] = __builtin_amdgcn_sdot4((int)a[0][0], w0.x, acc[r], false);
        acc[r] = __builtin_amdgcn_sdot4((int)a[0][1], w0.y, acc[r], false);
        acc[r] = __builtin_amdgcn_sdot4((int)a[0][2], w0.z, acc[r], false);
        acc[r] = __builtin_amdgcn_sdot4((int)a[1][0], w0.w, acc[r], false);
        acc[r] = __builtin_amdgcn_sdot4((int)a[1][1], w1.x, acc[r], false);
        acc[r] = __builtin_amdgcn_sdot4((int)a[1][2], w1.y, acc[r], false);
        acc[r] = __builtin_amdgcn_sdot4((int)a[2][0], w1.z, acc[r], false);
        acc[r] = __builtin_amdgcn_sdot4((int)a[2][1], w1.w, acc[r], false);
        acc[r] = __builtin_amdgcn_sdot4((int)a[2][2], w2, acc[r], false);
      }
      // four outputs at a time: |acc| < 2^21 here (at most 36 products of a byte and a signed byte, plus the
      // correction term), so the 24-bit multiplier gives the exact low 32 bits where the multipliers fit 24 bits
      bn_t kk[4], ll[4];
#pragma unroll
      for (int r = 0; r < 4; r++) {
        kk[r] = (MODE == EPI_BN) ? k_l[4 * n4 + r] : (bn_t)0;
        ll[r] = (MODE == EPI_BN) ? lam_l[4 * n4 + r] : (bn_t)0;
      }
      packed[n4] = requant4<MODE, true>(acc[0], acc[1], acc[2], acc[3], kk, ll, k_small, e.mult, e.shift);
    }
    if (m < g.M) {
      uint8_t *o = (uint8_t *)g.out + (long long)m * g.N;
      if (g.vec_store) {
        // N == NCH and 16-byte aligned rows: one copy of the store code per cache policy
        auto put = [&](auto nt) {
          constexpr bool NT = decltype(nt)::value;
#pragma unroll
          for (int q = 0; q < NCH / 16; q++)
            store16<NT>(o + 16 * q, (v4i){(int)packed[4 * q], (int)packed[4 * q + 1], (int)packed[4 * q + 2], (int)packed[4 * q + 3]});
        };
        if (g.nt) put(std::true_type{});
        else put(std::false_type{});
      } else {
#pragma unroll
        for (int n = 0; n < NCH; n++)
          if (n < g.N) o[n] = (uint8_t)(packed[n >> 2] >> (8 * (n & 3)));
      }
    }
    cur = nxt;
  }
}
