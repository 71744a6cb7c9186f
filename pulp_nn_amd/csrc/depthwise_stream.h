// 3x3 depthwise, CHW in, HWC out, streamed: a workgroup takes one image and 64 channels and walks down the
// whole plane, replacing 32bit/src/pulp_nn_depthwise_3x3_s1.c:103-223 and pulp_nn_depthwise_generic.c:138-179
// for planes of up to 64 output columns on whole 64-channel groups.
//
// Same arithmetic as dw3x3_lin_kernel (lane <-> channel, LDS channel stride odd, v_dot4 on byte windows with the
// (K0,K1,K2,0) / (0,K0,K1,K2) filters, activations as a ^ 0x80 applied as a dword is read from LDS with
// 128 * sum(w) added back, 4 x 4 byte transpose in each lane quad before the store).  What differs is the shape
// of the work:
//   * dw3x3_lin_kernel cuts a plane into bands of a few output rows, one workgroup each: every band stages
//     ky - sy input rows it shares with its neighbour, every wave restarts its partial sums at the top of every
//     band (two input rows of arithmetic that produce nothing), and every workgroup sets up its channels'
//     weights again.  Here a wave keeps the partial sums of its group of 4 output columns from the first row of
//     the plane to the last: each input row is staged once, multiplied once, and the per-channel set-up is done
//     once per plane.
//   * the plane's rows pass through LDS in chunks of CR rows, two chunk slots per channel.  Two loader waves
//     request chunk k + 1 (buffer loads that write LDS directly, one instruction per channel: a chunk of a
//     channel is contiguous in a CHW plane) while the computing waves work on chunk k; one barrier per chunk.
//     The computing waves never wait for memory: their stores are fire and forget, the loads belong to the
//     loader waves.
//   * the store addresses are a scalar row base plus a per-lane offset that never changes.
// How long the contiguous piece of a channel is that one request fetches decides the read rate (224-byte pieces:
// 37 us for the 56 x 56 x 128 stride-2 layer at batch 256, 448-byte pieces: 28 us), which is why a chunk is 8
// rows and not fewer; more than two workgroups' worth of LDS per compute unit costs more than it gains.
#pragma once
#include "depthwise.h"

#define DWS_LOADERS 2   // loader waves per workgroup (behind the computing waves)
#define DWS_ROWS 8      // input rows per chunk
#define DWS_AUX 2       // cache policy of the loads: nt (every input byte is read once)

// s_waitcnt vmcnt(n) for a run-time n: the instruction takes an immediate, so n is rounded down to a multiple of 8
// (waiting for fewer outstanding loads than allowed is always safe).  vmcnt is bits 3:0 and 15:14.
__device__ __forceinline__ void dws_wait_vm(int n)
{
#define DWS_VM(N) __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14))
  if (n >= 56) DWS_VM(56);
  else if (n >= 48) DWS_VM(48);
  else if (n >= 40) DWS_VM(40);
  else if (n >= 32) DWS_VM(32);
  else if (n >= 24) DWS_VM(24);
  else if (n >= 16) DWS_VM(16);
  else if (n >= 8) DWS_VM(8);
  else DWS_VM(0);
#undef DWS_VM
}

// Preconditions (checked by the host): W % 4 == 0, Wo % 4 == 0, Wo / 4 computing waves (at most 14) plus
// DWS_LOADERS loader waves per workgroup, CH % 64 == 0, input and output 4-byte aligned, B * CH * H * W < 2^31,
// PL as the template says; g.NR rows per chunk with g.NR * W % 16 == 0 and g.NR * W <= 1024, g.RB chunk slots per
// channel, g.CSD odd and at least g.RB * g.NR * W / 4 dwords, 4 * (64 * g.CSD + 8 * computing waves) bytes of LDS; g.cgroups =
// CH / 64, g.bands bands of output rows (every band at least one row; one band is the whole plane),
// g.total = B * g.bands * g.cgroups workgroups.
// The stores keep the default cache policy: a workgroup writes 64 of a pixel's channels, half a 128-byte line, and
// the other half comes from the neighbouring workgroup on the same XCD, so the line should stay in L2 until then.
template <int S, int PL, int MODE>
__global__ __launch_bounds__(1024, 8) void dw3x3_stream_kernel(DwGeom g, EpiArgs e)
{
  const int CR = g.NR;  // input rows per chunk: CR * W is a multiple of 16, a chunk of a channel is whole 16-byte pieces
  constexpr int O0 = 4 - PL;
  constexpr int NS = (O0 + 3 * S + 2) / 4 + 1;  // dwords per input row needed for 4 outputs
  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  extern __shared__ unsigned dw_lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nwc = (int)(blockDim.x >> 6) - DWS_LOADERS;  // computing waves = groups of 4 output columns
  const int LWD = g.LWD;                                  // = W / 4
  const int NSL = g.RB;                                   // chunk slots per channel in LDS (2 to 4)

  int id = dw_xcd_remap(blockIdx.x, g.total);
  const int cg = id % g.cgroups;
  id /= g.cgroups;
  const int band = id % g.bands, b = id / g.bands;
  const int c0 = cg * DW_CG;
  // The band's output rows o0 .. o1 - 1 read the padded input rows ipb .. ipb + PR - 1 (padded row ip is image row
  // ip - pt); of those, image rows iy0 .. iy0 + nreal - 1 exist, the others are zeros.  In band coordinates
  // (ip counted from the band's first padded row) the real rows are ip = ztop .. ztop + nreal - 1.
  const int hob = (g.Ho + g.bands - 1) / g.bands;
  const int o0 = band * hob, nho = min(g.Ho, o0 + hob) - o0;
  const int ipb = o0 * S;
  const int PR = (nho - 1) * S + 3;
  const int iy0 = max(0, ipb - g.pt), ztop = max(0, g.pt - ipb);
  const int nreal = max(0, min(g.H, ipb + PR - g.pt) - iy0);  // (0: a band that lies in the padding altogether)
  const int nck = (nreal + CR - 1) / CR;  // chunks of the band

  if (wave >= nwc) {
    // ---- loader waves: chunk k of channel c = rows k*CR .. of its plane, contiguous; lane l fetches the 16-byte
    // piece l of it.  Pieces past the end of the plane are never read (rows past the image are supplied as zeros
    // by the computing waves); past the end of the input they are out of range and load zeros.
    const int lw = wave - nwc;
    const __amdgpu_buffer_rsrc_t rsrc_in =
        __builtin_amdgcn_make_buffer_rsrc((void *)g.in, 0, (unsigned)(g.planes * g.H * g.W), 0x00020000);
    // (one instruction per channel and chunk: the host keeps a chunk within the 1 KB a wave's load covers)
    auto request = [&](int k) {
      const int slot = k % NSL;
      const int bytes = min(CR, nreal - k * CR) * g.W;  // the last chunk may be short: nothing is fetched past it
      if (16 * lane < bytes) {
#pragma unroll 4
        for (int c = lw; c < DW_CG; c += DWS_LOADERS) {
          const int soff = ((b * g.CH + c0 + c) * g.H + iy0 + k * CR) * g.W;
          unsigned *dst = dw_lds + c * g.CSD + slot * (CR * LWD);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_in, (lds_ptr_t)dst, 16, 16 * lane, soff, 0, DWS_AUX);
        }
      }
    };
    // Barrier k (k = 0 .. nck - 1) stands before the computing waves' work on chunk k; every wave of the workgroup
    // passes exactly nck barriers.  The first NSL chunks are requested at once; a chunk's slot is free again once
    // the chunk is consumed, that is behind the next barrier, so chunk k - 1 + NSL is requested behind barrier k.
    // Before this wave arrives at barrier k, chunk k has landed: loads return in order, so that is "at most the
    // requests of the chunks behind k are outstanding", a request being `per` instructions for this wave.
    const int per = (DW_CG - lw + DWS_LOADERS - 1) / DWS_LOADERS;
    int next = min(NSL, nck);
    for (int k = 0; k < next; k++) request(k);
    for (int k = 0; k < nck; k++) {
      dws_wait_vm((next - 1 - k) * per);
      __builtin_amdgcn_s_barrier();
      if (k >= 1 && next < nck) request(next++);
    }
    return;
  }

  // ---- computing waves: per-lane channel constants ------------------------------------------------
  const int ch = c0 + lane;
  unsigned wA[3], wB[3];
  int wsum = 0;
#pragma unroll
  for (int i = 0; i < 3; i++) {
    const int8_t *p = g.wt + (long long)ch * 9 + 3 * i;
    const unsigned k0 = (uint8_t)p[0], k1 = (uint8_t)p[1], k2 = (uint8_t)p[2];
    wA[i] = k0 | (k1 << 8) | (k2 << 16);
    wB[i] = wA[i] << 8;
    wsum += (int)p[0] + (int)p[1] + (int)p[2];
  }
  const int corr = 128 * wsum + (g.bias ? (int)g.bias[ch] : 0);
  const bn_t kk = MODE == EPI_BN ? e.k[ch] : (bn_t)0, ll = MODE == EPI_BN ? e.lambda[ch] : (bn_t)0;
  const bool fastq = (MODE == EPI_BN) ? __all(bn_k_small(kk)) : (e.shift >= 16);
  const unsigned sel1 = quad_sel1(lane), sel2 = quad_sel2(lane);

  const int xg = wave;
  const int dc0 = xg * S - 1;  // dword column of the first dword of the window
  const bool edge = dc0 < 0 || dc0 + NS > LWD;
  const unsigned *lbase = dw_lds + lane * g.CSD + dc0;
  // 8 zero dwords per computing wave behind the staged rows (written and read by this wave only)
  unsigned *zeros = dw_lds + DW_CG * g.CSD + 8 * wave;
  if (lane < 8) zeros[lane] = 0;
  // output: scalar row base + this lane's offset (pixel lane % 4 of the group, channels 4 * (lane / 4) ..)
  uint8_t *orow = g.out + (((long long)b * g.Ho + o0) * g.Wo + 4 * xg) * g.CH + c0;
  const unsigned voff = (unsigned)(lane & 3) * (unsigned)g.CH + (unsigned)(lane & ~3);
  const long long row_bytes = (long long)g.Wo * g.CH;

  auto walk = [&](auto edge_tag, auto fast_tag) {
    constexpr bool EDGE = decltype(edge_tag)::value, FASTQ = decltype(fast_tag)::value;
    // Dwords of the window that lie left or right of the row (first and last group of columns only) are read from a
    // dword of the window that does exist and masked to zero activations; rows above and below the image are read
    // from a few zero dwords that each wave keeps behind the staged rows.  The loop itself has no branch for either.
    int dsub[NS];
    unsigned dmask[NS];
#pragma unroll
    for (int d = 0; d < NS; d++) {
      const bool in_row = !EDGE || (dc0 + d >= 0 && dc0 + d < LWD);
      dsub[d] = in_row ? d : 1;  // dword 1 of a window is inside the row for every group of columns
      dmask[d] = in_row ? 0xFFFFFFFFu : 0u;
    }
    auto read_row = [&](const unsigned *p, unsigned (&span)[NS]) {
#pragma unroll
      for (int d = 0; d < NS; d++) {
        if constexpr (EDGE) span[d] = (p[dsub[d]] & dmask[d]) ^ 0x80808080u;
        else span[d] = p[d] ^ 0x80808080u;
      }
    };
    auto taps = [&](const unsigned (&span)[NS], int i, int (&acc)[4]) {
      dw_tap<O0, NS>(span, wA[i], wB[i], acc[0]);
      dw_tap<O0 + S, NS>(span, wA[i], wB[i], acc[1]);
      dw_tap<O0 + 2 * S, NS>(span, wA[i], wB[i], acc[2]);
      dw_tap<O0 + 3 * S, NS>(span, wA[i], wB[i], acc[3]);
    };
    auto taps_first = [&](const unsigned (&span)[NS], int (&acc)[4]) {
      acc[0] = dw_tap_first<O0, NS>(span, wA[0], wB[0], corr);
      acc[1] = dw_tap_first<O0 + S, NS>(span, wA[0], wB[0], corr);
      acc[2] = dw_tap_first<O0 + 2 * S, NS>(span, wA[0], wB[0], corr);
      acc[3] = dw_tap_first<O0 + 3 * S, NS>(span, wA[0], wB[0], corr);
    };
    auto emit = [&](int (&acc)[4]) {
      unsigned packed = requant4_same<MODE, FASTQ>(acc[0], acc[1], acc[2], acc[3], kk, ll, e.mult, e.shift);
      packed = quad_transpose4x4_perm(packed, sel1, sel2);
      store4<false>(orow + voff, (int)packed);
      orow += row_bytes;
    };
    // Partial sums.  With stride 1 the padded input row ip starts output row ip (filter row 0), is the middle row
    // of output ip - 1 and finishes output ip - 2: three sets F, M, N that hand their contents on after every row
    // (the compiler renames registers over the three rows of the unrolled loop, no copies remain).  With stride 2
    // output o starts at ip = 2o, has its middle row at 2o + 1 and ends at 2o + 2, where output o + 1 starts
    // from the same row: one set.
    int F[4] = {0, 0, 0, 0}, M[4] = {0, 0, 0, 0}, N[4] = {0, 0, 0, 0};
    // CHK: near the top and the bottom of the plane, test which of the roles exist; ODD (stride 2): ip is odd
    auto row = [&](auto chk_tag, auto odd_tag, int ip, const unsigned (&span)[NS]) {
      constexpr bool CHK = decltype(chk_tag)::value, ODD = decltype(odd_tag)::value;
      if constexpr (S == 1) {
        if (!CHK || ip >= 2) {
          taps(span, 2, F);
          emit(F);
        }
        if (!CHK || (ip >= 1 && ip - 1 < nho)) taps(span, 1, M);
        if (!CHK || ip < nho) taps_first(span, N);
#pragma unroll
        for (int j = 0; j < 4; j++) {
          F[j] = M[j];
          M[j] = N[j];
        }
      } else if constexpr (ODD) {
        taps(span, 1, N);
      } else {
        if (!CHK || ip >= 2) {
          taps(span, 2, N);
          emit(N);
        }
        if (!CHK || ip / 2 < nho) taps_first(span, N);
      }
    };
    constexpr int PER = S == 1 ? 3 : 4;  // rows per turn of the unrolled loop
    const std::true_type yes{};
    const std::false_type no{};

    // segment -1: the padded rows above the image; 0 .. nck - 1: the chunks; nck: the padded rows below
    for (int k = -1; k <= nck; k++) {
      const bool real = k >= 0 && k < nck;
      int ip, ip1;
      if (k < 0) ip = 0, ip1 = min(ztop, PR);
      else if (k < nck) ip = k * CR + ztop, ip1 = min(min((k + 1) * CR, nreal) + ztop, PR);
      else ip = min(nreal + ztop, PR), ip1 = PR;
      if (real) __builtin_amdgcn_s_barrier();  // B_k: chunk k has landed, everybody is done with chunk k - 1
      const unsigned *p = real ? lbase + (k % NSL) * (CR * LWD) : zeros;
      const int pinc = real ? LWD : 0;
      unsigned span[NS];
      auto one = [&](auto chk_tag, auto odd_tag) {
        read_row(p, span);
        p += pinc;
        row(chk_tag, odd_tag, ip, span);
        ip++;
      };
      // away from the top and the bottom of the plane every role exists
      if constexpr (S == 1) {
        while (ip + PER <= ip1 && ip >= 2 && ip + PER - 1 < nho) {
          one(no, no);
          one(no, no);
          one(no, no);
        }
      } else if (ip & 1) {
        while (ip + PER <= ip1 && ip >= 2 && (ip + PER - 1) / 2 < nho) {
          one(no, yes);
          one(no, no);
          one(no, yes);
          one(no, no);
        }
      } else {
        while (ip + PER <= ip1 && ip >= 2 && (ip + PER - 1) / 2 < nho) {
          one(no, no);
          one(no, yes);
          one(no, no);
          one(no, yes);
        }
      }
      while (ip < ip1) {
        if (S == 2 && (ip & 1)) one(yes, yes);
        else one(yes, no);
      }
    }
  };
  if (fastq) {
    if (edge) walk(std::true_type{}, std::true_type{});
    else walk(std::false_type{}, std::true_type{});
  } else {
    if (edge) walk(std::true_type{}, std::false_type{});
    else walk(std::false_type{}, std::false_type{});
  }
}
