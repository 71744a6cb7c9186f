// Max / average pooling and element-wise add on HWC uint8 maps: bandwidth-bound
// VALU kernels, one thread per output pixel and group of 4 channels (16 for
// add), so that neighbouring lanes read and write neighbouring bytes.
#pragma once
#include "memops.h"
#include "requant.h"

typedef unsigned short ushort2v __attribute__((ext_vector_type(2)));

// per-byte unsigned max of two packed dwords (v_pk_max_u16 on even and odd bytes)
__device__ __forceinline__ unsigned max_u8x4(unsigned a, unsigned b)
{
  const unsigned m = 0x00FF00FFu;
  unsigned ae = a & m, be = b & m, ao = (a >> 8) & m, bo = (b >> 8) & m;
  ushort2v e = __builtin_elementwise_max(*(ushort2v *)&ae, *(ushort2v *)&be);
  ushort2v o = __builtin_elementwise_max(*(ushort2v *)&ao, *(ushort2v *)&bo);
  return *(unsigned *)&e | (*(unsigned *)&o << 8);
}

struct PoolGeom {
  const uint8_t *in;
  uint8_t *out;
  int B, H, W, C, Ho, Wo;
  int kx, ky, sx, sy;
  int pt, pb, pl, pr;
  int cgroups;   // ceil(C / 4)
  int vec4;      // pointers and C are multiples of 4
  long long total;  // B * Ho * Wo * cgroups threads
};

__device__ __forceinline__ unsigned load4(const uint8_t *p, int n, int vec4)
{
  if (vec4) return *(const unsigned *)p;
  unsigned v = 0;
  for (int j = 0; j < n; j++) v |= (unsigned)p[j] << (8 * j);
  return v;
}

__device__ __forceinline__ void store4(uint8_t *p, unsigned v, int n, int vec4)
{
  if (vec4) {
    *(unsigned *)p = v;
    return;
  }
  for (int j = 0; j < n; j++) p[j] = (uint8_t)(v >> (8 * j));
}

// pulp_nn_maxpool (32bit/src/pulp_nn_maxpool.c:27-146): unsigned max over the
// window [ox*sx - pl, +kx) x [oy*sy - pt, +ky) clamped to the image.  The
// reference computes it as an in-place x pass followed by a y pass and
// overwrites its input; this kernel reads the input once and leaves it intact.
__global__ __launch_bounds__(256) void maxpool_kernel(PoolGeom g)
{
  long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= g.total) return;
  const int cg = (int)(t % g.cgroups);
  t /= g.cgroups;
  const int ox = (int)(t % g.Wo);
  t /= g.Wo;
  const int oy = (int)(t % g.Ho);
  const int b = (int)(t / g.Ho);
  const int c = cg * 4, n = min(4, g.C - c);
  const int xs = max(ox * g.sx - g.pl, 0), xe = min(ox * g.sx - g.pl + g.kx, g.W);
  const int ys = max(oy * g.sy - g.pt, 0), ye = min(oy * g.sy - g.pt + g.ky, g.H);
  const uint8_t *img = g.in + (long long)b * g.H * g.W * g.C + c;
  unsigned m = 0;
  for (int y = ys; y < ye; y++)
    for (int x = xs; x < xe; x++) m = max_u8x4(m, load4(img + ((long long)y * g.W + x) * g.C, n, g.vec4));
  store4(g.out + (((long long)b * g.Ho + oy) * g.Wo + ox) * g.C + c, m, n, g.vec4);
}

// Same, 16 channels per thread with 16-byte accesses (C % 16 == 0, 16-byte aligned maps).
// g.cgroups counts groups of 16 here.  NT: non-temporal store; LNT: non-temporal loads (windows that do not
// overlap on an input too large for the caches: every byte is read once).  A whole 2 x 2 window is four loads
// issued together; other windows go tap by tap.
template <bool NT, bool LNT>
__global__ __launch_bounds__(256) void maxpool16_kernel(PoolGeom g)
{
  long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= g.total) return;
  const int cg = (int)(t % g.cgroups);
  t /= g.cgroups;
  const int ox = (int)(t % g.Wo);
  t /= g.Wo;
  const int oy = (int)(t % g.Ho);
  const int b = (int)(t / g.Ho);
  const int xs = max(ox * g.sx - g.pl, 0), xe = min(ox * g.sx - g.pl + g.kx, g.W);
  const int ys = max(oy * g.sy - g.pt, 0), ye = min(oy * g.sy - g.pt + g.ky, g.H);
  const uint8_t *img = g.in + (long long)b * g.H * g.W * g.C + cg * 16;
  auto ld = [&](const uint8_t *p) { return LNT ? __builtin_nontemporal_load((const v4i *)p) : *(const v4i *)p; };
  auto vmax = [&](v4i &m, const v4i &v) {
    m.x = (int)max_u8x4((unsigned)m.x, (unsigned)v.x);
    m.y = (int)max_u8x4((unsigned)m.y, (unsigned)v.y);
    m.z = (int)max_u8x4((unsigned)m.z, (unsigned)v.z);
    m.w = (int)max_u8x4((unsigned)m.w, (unsigned)v.w);
  };
  v4i m = {0, 0, 0, 0};
  if (ye - ys == 2 && xe - xs == 2) {
    const uint8_t *p = img + ((long long)ys * g.W + xs) * g.C;
    const long long row = (long long)g.W * g.C;
    const v4i v0 = ld(p), v1 = ld(p + g.C), v2 = ld(p + row), v3 = ld(p + row + g.C);
    m = v0;
    vmax(m, v1);
    vmax(m, v2);
    vmax(m, v3);
  } else {
    for (int y = ys; y < ye; y++)
      for (int x = xs; x < xe; x++) vmax(m, ld(img + ((long long)y * g.W + x) * g.C));
  }
  store16<NT>(g.out + (((long long)b * g.Ho + oy) * g.Wo + ox) * g.C + cg * 16, m);
}

// pulp_nn_avgpool (32bit/src/pulp_nn_avgpool.c:29-121): window bounds exactly as
// written there (:82-86: the y start uses padding_b, the x end uses padding_r),
// divisor always kx*ky, and the requantisation in uint32_t (32-bit tree, :106-110)
// or int64_t with low-32 truncation by the clip (64-bit tree).
struct AvgArgs {
  long long lambda, out_add;
  int shift, requant;
};

__global__ __launch_bounds__(256) void avgpool_kernel(PoolGeom g, AvgArgs a)
{
  long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= g.total) return;
  const int cg = (int)(t % g.cgroups);
  t /= g.cgroups;
  const int ox = (int)(t % g.Wo);
  t /= g.Wo;
  const int oy = (int)(t % g.Ho);
  const int b = (int)(t / g.Ho);
  const int c = cg * 4, n = min(4, g.C - c);
  const int ys = max(0, oy * g.sy - g.pb), ye = min(oy * g.sy - g.pt + g.ky, g.H);
  const int xs = max(0, ox * g.sx - g.pl), xe = min(ox * g.sx - g.pr + g.kx, g.W);
  const uint8_t *img = g.in + (long long)b * g.H * g.W * g.C + c;
  unsigned sum[4] = {0, 0, 0, 0};
  // four taps at a time, their loads issued together (taps past the window re-read its last
  // column and are not counted): one load per round trip would make the window size the
  // kernel's latency
  for (int y = ys; y < ye; y++)
    for (int x = xs; x < xe; x += 4) {
      unsigned v[4];
#pragma unroll
      for (int i = 0; i < 4; i++) v[i] = load4(img + ((long long)y * g.W + min(x + i, xe - 1)) * g.C, n, g.vec4);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        if (x + i < xe) {
#pragma unroll
          for (int j = 0; j < 4; j++) sum[j] += (v[i] >> (8 * j)) & 0xFF;
        }
      }
    }
  const unsigned ksize = (unsigned)(g.kx * g.ky);
  unsigned packed = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    int res;
    if (a.requant) {
#if PULPNN_BN_BITS == 64
      long long v = (long long)((unsigned long long)sum[j] * (unsigned long long)a.lambda);
      v = v / (long long)ksize;
      v = (long long)((unsigned long long)v + (unsigned long long)a.out_add);
      res = (int)(unsigned)(unsigned long long)(v >> a.shift);
#else
      unsigned v = sum[j] * (unsigned)(int)a.lambda / ksize + (unsigned)(int)a.out_add;
      res = (int)(v >> a.shift);
#endif
    } else {
      res = (int)(sum[j] / ksize);
    }
    packed |= (unsigned)clipu8(res) << (8 * j);
  }
  store4(g.out + (((long long)b * g.Ho + oy) * g.Wo + ox) * g.C + c, packed, n, g.vec4);
}

// pulp_nn_add (32bit/src/pulp_nn_add.c:27-62) with pulp_nn_add_quant_u8
// (32bit/src/pulp_nn_utils.c:47-60): min(255, (uint16)((uint32)(a*m1 + b*m2) >> d)).
__device__ __forceinline__ unsigned add_quant4(unsigned a, unsigned b, int m1, int m2, int d)
{
  unsigned r = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const unsigned v = (unsigned)((int)((a >> (8 * j)) & 0xFF) * m1 + (int)((b >> (8 * j)) & 0xFF) * m2);
    r |= min((v >> d) & 0xFFFFu, 255u) << (8 * j);
  }
  return r;
}

__global__ __launch_bounds__(256) void add_kernel(const uint8_t *a, const uint8_t *b, uint8_t *out, long long n,
                                                  int m1, int m2, int d, int vec16)
{
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long i = t * 16;
  if (i >= n) return;
  if (vec16 && i + 16 <= n) {
    const uint4 va = *(const uint4 *)(a + i), vb = *(const uint4 *)(b + i);
    uint4 r;
    r.x = add_quant4(va.x, vb.x, m1, m2, d);
    r.y = add_quant4(va.y, vb.y, m1, m2, d);
    r.z = add_quant4(va.z, vb.z, m1, m2, d);
    r.w = add_quant4(va.w, vb.w, m1, m2, d);
    *(uint4 *)(out + i) = r;
  } else {
    for (long long j = i; j < min(i + 16, n); j++) {
      const unsigned v = (unsigned)((int)a[j] * m1 + (int)b[j] * m2);
      out[j] = (uint8_t)min((v >> d) & 0xFFFFu, 255u);
    }
  }
}
