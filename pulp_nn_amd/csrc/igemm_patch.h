// Implicit-GEMM kernel for large 3-wide, stride-1 convolutions on images up to 64 output columns wide: the
// MFMA-bound case of 32bit/src/pulp_nn_conv_Ho_parallel.c:76-183 + pulp_nn_matmul.c:53-216, with the im2col
// reuse of the reference's pulp_nn_im2col step (conv_Ho_parallel.c:100-140) turned inside out: there a pixel's
// patch is copied once per pixel, here an input row is staged once per filter row and read three times.
//
// Same arithmetic, operand path (buffer loads that write LDS, XOR swizzle on the global address), weight sums by
// MFMA, persistent workgroups, folded epilogue constants and register pipelining as igemm_ring_kernel.  What
// differs is the pixel tile and what a stage of LDS holds:
//   * igemm_ring_kernel's tile is 256 consecutive output pixels, and every filter tap is a K sub-slice of its own:
//     256 rows x 64 bytes of activations per tap and 64 input channels, although the three taps of one filter
//     row read the same input pixels shifted by one column;
//   * here the tile is a patch of 4 output rows x 64 columns.  For a filter row fy and 64 input channels the input
//     pixels behind it are 4 rows of 66 columns (a halo column each side): they are staged once, as 4 x 72 LDS rows
//     (row = 72 * tile row + column + 1; the 6 spare rows per tile row keep the row number of a pixel congruent to
//     its column modulo 8, which the swizzle needs), and the fragments of tap fx are the same rows read at
//     column offset fx, an immediate in the LDS read.  Zero padding needs no per-lane work: a halo column or a row
//     outside the image is an out-of-range load, which writes zeros.  Activation bytes from L2 per filter row and
//     64 channels: 264 rows against 3 x 256.
//   * a group = the three sub-slices (fx = 0, 1, 2) of one filter row and 64 input channels: one activation
//     block (18 KB) and three weight sub-slices (16 KB each).  LDS holds three activation blocks and two sets of
//     weight sub-slices.  While group j is multiplied, group j + 1 has landed or is landing, and group j + 2 is
//     requested at the last sub-slice of group j, behind the one barrier a group needs: its weights take the
//     place of group j's (read a sub-slice ago), its activations that of group j - 1's, so the activation
//     fragments of the sub-slice being multiplied can still be read behind the barrier;
//   * which is what frees registers: only four activation fragments are held, not eight.  Fragment s + 4 of the
//     current sub-slice is read into the registers of fragment s when that one's MFMAs are issued, fragment s of
//     the next sub-slice into those of fragment s + 4: every read is four MFMA groups (64 MFMAs of the two waves
//     of a SIMD) ahead of its use.
// Output pixels outside the image (column 63 when Wo = 63, rows past Ho) are computed and not stored; the host
// takes this kernel only when at least nine tenths of the patch grid are real pixels.
//
// Measured on the 64 x 64 x 256 -> 256 layer at batch 64 (conv_phases tool, both kernels in one run, output equal byte
// for byte): 31 % fewer bytes from L2, 3 % less time in the main loop, the launch 1 to 2 % shorter than
// igemm_ring_kernel's (142 against 144 us).  The layer runs at the power limit (shader clock 2.0 to 2.1 GHz inside
// the loop against 2.4 GHz for the same loop on zeros), so the saved traffic comes back as a little more clock.
// Preconditions (checked by the host): kx = 3, stride 1, pl <= 1, Wo <= 64, ky <= 31, ky * Ci / 64 >= 2 groups,
// Ci % 64 = 0, N % 16 = 0, whole images, a grid that is a multiple of 8 * tiles_n and no larger than the number of
// tiles, g.rgroups = ceil(Ho / 4) with its divisor.
#pragma once
#include "igemm_ring.h"

#define IGP_PITCH 72                                 // LDS rows per tile row
#define IGP_A_BYTES (4 * IGP_PITCH * 64)             // activation block of a group
#define IGP_A_BLOCKS (IGP_A_BYTES / 1024)            // in 16-row loads: 18
#define IGP_W_BYTES (256 * 64)                       // one weight sub-slice
#define IGP_W_BASE (3 * IGP_A_BYTES)                 // three activation blocks, then two sets of three weight sub-slices
#define IGP_W_SET (3 * IGP_W_BYTES)
#define IGP_DUMP_AT (IGP_W_BASE + 2 * IGP_W_SET)     // 1 KB where loads without a destination go
#define IGP_DUMP 1024
#define IGP_THREADS 512
#define IGP_BN 256

static inline int igp_lds_bytes() { return IGP_DUMP_AT + IGP_DUMP + IGP_BN * (4 + 2 * (int)sizeof(bn_t)); }

// ABL (tools only, wrong results): 1 = no loads after a tile's first two groups, 2 = one MFMA per sub-slice,
// 4 = no fragment reads in the loop, 8 = no epilogue, 16 = epilogue without its stores, 32 = activation loads out of
// range (zeros written, nothing fetched), 64 = weight loads out of range.
template <int MODE, int ABL = 0>
__global__ __launch_bounds__(IGP_THREADS, 1) void igemm_patch_kernel(ConvGeom g, EpiArgs e)
{
  constexpr int TM = 8, TN = 4, WNC = 64, BN = IGP_BN, GA = 3, GW = 2;
  constexpr int G = GA + 3 * GW;  // loads per wave and group
  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char igr_lds[];
  int *wsum = (int *)(igr_lds + IGP_DUMP_AT + IGP_DUMP);  // weight sums by LDS row
  bn_t *cadd = (bn_t *)(wsum + BN);      // per channel: additive constant of the epilogue
  bn_t *cmul = cadd + BN;                // per channel: multiplier (batch-norm branch)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave & 1, wave_n = wave >> 1;
  const int l16 = lane & 15, lgrp = lane >> 4;

  // tiles of this workgroup: t, t + gridDim.x, ... (a multiple of 8 * tiles_n apart: same channel range; an XCD
  // gets a contiguous range of tiles).  No early exit, see igemm_ring_kernel.
  int tile = (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3);
  auto tile_m_of = [&](int t) { return (int)fastdiv((unsigned)t, g.d_tiles_n); };
  const int n0 = (tile - tile_m_of(tile) * g.tiles_n) * BN;

  const unsigned OOB = 0x80000000u;
  const unsigned shift = (unsigned)((g.pt * g.W + g.pl) * g.Ci);
  const __amdgpu_buffer_rsrc_t rsrc_a =
      __builtin_amdgcn_make_buffer_rsrc((void *)(g.in - shift), 0, shift + (unsigned)g.batch * (unsigned)g.in_img, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)g.w, 0, (unsigned)g.N * (unsigned)g.K, 0x00020000);

  // ---- what this lane fetches ------------------------------------------------------------------
  // A load fills 16 LDS rows: lane l writes slot l%4 of row l/4 of the block, which has to hold K chunk
  // (l%4) ^ ((row/2)%4).  Weights: wave w loads blocks 2w, 2w+1 of each sub-slice, rows in fragment order as in
  // igemm_ring_kernel.  Activations: wave w loads blocks w, w + 8, w + 16 of the group's block (those past the
  // 18th go to the dump area, out of range: the number of loads per wave stays the same).
  // (Everything this lane needs for the loads and the fragment reads is derived from an opaque copy of the lane
  // number, once before a tile's first loads and again at the top of its main loop.  Derived from the lane number
  // itself these values would be loop invariants, kept in registers across the epilogue, which has none to spare:
  // they would be spilled there and reloaded inside the main loop, behind the loads in flight.)
  unsigned poff[GA], pinv[GA], woff;
  auto weight_setup = [&]() {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    // (the second block's rows are 16 LDS rows further: the next t of the fragment order, 4 channels further, in
    // the same group of 16 channels; that is 4 * K bytes, added to the loads' scalar offset)
    const int row = 16 * (GW * wave) + (ln >> 2);
    const unsigned chunk = (unsigned)((ln & 3) ^ ((row >> 1) & 3));
    const int pp = row % WNC, t = pp >> 4, r16 = pp & 15;
    const int n = n0 + (row / WNC) * WNC + (r16 >> 2) * (4 * TN) + 4 * t + (r16 & 3);
    woff = n < g.N ? (unsigned)n * (unsigned)g.K + 16u * chunk : OOB;
  };
  // tile tm = image b, output rows oy0 .. oy0 + 3, all columns
  int oy0 = 0, img = 0;
  auto pixel_setup = [&](int tm) {
    img = (int)fastdiv((unsigned)tm, g.d_rg);
    oy0 = 4 * (tm - img * g.rgroups);
    int ln = lane;
    asm volatile("" : "+v"(ln));
#pragma unroll
    for (int j = 0; j < GA; j++) {
      const int beta = wave + 8 * j;
      const int rho = 16 * beta + (ln >> 2);
      const unsigned chunk = (unsigned)((ln & 3) ^ ((rho >> 1) & 3));
      const int ry = rho / IGP_PITCH, cx = rho - ry * IGP_PITCH;  // input column cx - pl
      const bool live = beta < IGP_A_BLOCKS && cx < g.Wo + 2 && (unsigned)(cx - g.pl) < (unsigned)g.W && img < g.batch;
      poff[j] = (unsigned)img * (unsigned)g.in_img + (unsigned)(((oy0 + ry) * g.W + cx) * g.Ci) + 16u * chunk;
      // filter rows fy with input row iy0 + fy inside the image: fy_lo <= fy < fy_hi, one bit each (ky <= 31)
      const int iy0 = oy0 + ry - g.pt;
      const int fy_lo = max(-iy0, 0), fy_hi = min(g.H - iy0, g.ky);
      const unsigned valid = fy_hi > fy_lo ? (1u << fy_hi) - (1u << fy_lo) : 0u;
      pinv[j] = live ? ~valid : ~0u;
    }
  };

  // The next group to request: filter row fy = group / (Ci / 64), channels 64 * (group % (Ci / 64)) ..; computed
  // from the counter with scalar multiply-high divisions (see igemm_ring_kernel).
  int u_group = 0;
  const int NG = g.ky * g.cpt;
  // group u_group -> activation block u_group % 3, weight set u_group % 2 (u_a, u_w)
  int u_a = 0, u_w = 0;
  auto dma = [&](unsigned dead) {
    const unsigned fy = fastdiv((unsigned)u_group, g.d_cpt);
    const unsigned ci = ((unsigned)u_group - fy * (unsigned)g.cpt) * 64u;
    const int fy_s = __builtin_amdgcn_readfirstlane((int)fy);
    const int soff_a = __builtin_amdgcn_readfirstlane((int)(fy * (unsigned)g.W * (unsigned)g.Ci + ci));
    const int soff_w = __builtin_amdgcn_readfirstlane((int)(fy * (unsigned)g.kx * (unsigned)g.Ci + ci));
#pragma unroll
    for (int j = 0; j < GA; j++) {
      const int beta = wave + 8 * j;
      unsigned char *dst = igr_lds + (beta < IGP_A_BLOCKS ? u_a * IGP_A_BYTES + 1024 * beta : IGP_DUMP_AT);
      const unsigned oob = ((unsigned)__builtin_amdgcn_sbfe((int)pinv[j], fy_s, 1) & OOB) | dead | ((ABL & 32) ? OOB : 0u);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)dst, 16, (int)(poff[j] | oob), soff_a, 0, 0);
    }
    unsigned char *w_dst = igr_lds + IGP_W_BASE + u_w * IGP_W_SET + wave * (1024 * GW);
#pragma unroll
    for (int fx = 0; fx < 3; fx++)
#pragma unroll
      for (int j = 0; j < GW; j++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr_t)(w_dst + fx * IGP_W_BYTES + 1024 * j), 16, (int)(woff | dead | ((ABL & 64) ? OOB : 0u)),
                                                 soff_w + fx * g.Ci + j * 4 * g.K, 0, 0);
    u_group++;
    u_a = u_a == 2 ? 0 : u_a + 1;
    u_w = 1 - u_w;
  };
  auto first_loads = [&]() {
    u_group = u_a = u_w = 0;  // (the host guarantees NG >= 2)
    dma(0u);
    dma(0u);
  };

  // Fragment addresses of this lane.  Activations: the pixel of fragment s, lane l16 is tile row
  // 2 * wave_m + s / 4, column 16 * (s % 4) + l16, and tap fx reads LDS row 72 * tile row + column + fx =
  // c + l16 with c = 72 * (s / 4) + 16 * (s % 4) + fx (+ 144 * wave_m): c = fx (mod 8), so the slot of chunk lgrp,
  // lgrp ^ (((c + l16) / 2) % 4), depends on fx and the lane only, and 64 * c is an immediate.
  int a_lane[3], w_lane;
  auto fragment_setup = [&]() {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int l16_ = ln & 15, lgrp_ = ln >> 4;
#pragma unroll
    for (int fx = 0; fx < 3; fx++)
      a_lane[fx] = wave_m * (2 * IGP_PITCH * 64) + l16_ * 64 + ((lgrp_ ^ (((fx + l16_) >> 1) & 3)) << 4);
    w_lane = IGP_W_BASE + (wave_n * WNC + l16_) * 64 + ((lgrp_ ^ ((l16_ >> 1) & 3)) << 4);
  };
  auto a_imm = [](int s, int fx) { return ((s / 4) * IGP_PITCH + 16 * (s % 4) + fx) * 64; };

  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
  v4i acc[TN][TM];
  v4i wacc[2];

  weight_setup();
  fragment_setup();
  pixel_setup(tile_m_of(tile));
  first_loads();

  bool first = true;
  [[maybe_unused]] int round = 0;
#pragma unroll 1
  for (; tile < g.tiles_total; tile += gridDim.x) {
    const int cur_oy0 = oy0, cur_img = img;
    IGR_STAMP(0)
#pragma unroll
    for (int t = 0; t < TN; t++)
#pragma unroll
      for (int s = 0; s < TM; s++) acc[t][s] = (v4i){0, 0, 0, 0};
    wacc[0] = wacc[1] = (v4i){0, 0, 0, 0};

    auto main_loop = [&](auto ws_tag) {
      constexpr bool WS = decltype(ws_tag)::value;
      v4i af[4], w0[TN], w1[TN];
      // Sub-slice FX of group grp (activation block ab, weight set ws): multiply its fragments and read ahead.
      // Activation fragment s sits in af[s % 4]: when the MFMAs of fragment s < 4 are issued its registers take
      // fragment s + 4 of this sub-slice, those of fragment s >= 4 take fragment s - 4 of the next sub-slice (FX + 1
      // of this group, or tap 0 of the next group); the weight fragments of the next sub-slice are read with the
      // first four.
      // At FX = 2, first: no load of this wave is outstanding (the next group has landed) and every LDS read it
      // issued is back; behind the barrier both hold for every wave, and the group after the next is requested:
      // into this group's weight set (last read a sub-slice ago) and the previous group's activation block.
      auto step = [&](auto fx_tag, v4i (&wc)[TN], v4i (&wn)[TN], int grp, int ab, int ws) {
        constexpr int FX = decltype(fx_tag)::value;
        constexpr int NFX = FX == 2 ? 0 : FX + 1;
        if constexpr (FX == 2) {
          IGR_WAIT(0, 1);
          __builtin_amdgcn_s_barrier();
          if (!(ABL & 1)) dma(grp + 2 < NG ? 0u : OOB);
        }
        const unsigned char *ca = igr_lds + ab * IGP_A_BYTES;
        const unsigned char *na = FX == 2 ? igr_lds + (ab == 2 ? 0 : ab + 1) * IGP_A_BYTES : ca;
        const unsigned char *nw = igr_lds + (FX == 2 ? 1 - ws : ws) * IGP_W_SET + NFX * IGP_W_BYTES;
#pragma unroll
        for (int s = 0; s < TM; s++) {
          const v4i a = af[s % 4] ^ (int)0x80808080;
#pragma unroll
          for (int t = 0; t < TN; t++)
            if (!(ABL & 2) || (s == 0 && t == 0)) acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wc[t], a, acc[t][s], 0, 0, 0);
          if (!(ABL & 4)) {
            if (s < 4) {
              af[s] = *(const v4i *)(ca + a_lane[FX] + a_imm(s + 4, FX));
              wn[s] = *(const v4i *)(nw + w_lane + s * 1024);
            } else {
              af[s - 4] = *(const v4i *)(na + a_lane[NFX] + a_imm(s - 4, NFX));
            }
          } else if (s < 4) {
            wn[s] = wc[s];
          }
          // keep the instructions of a fragment together and the fragments in this order: left to itself the
          // scheduler puts all the xors in front of the first MFMA and sinks the reads to the end of the iteration
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (WS) {
          const v4i ws0 = wave_m ? wc[2] : wc[0], ws1 = wave_m ? wc[3] : wc[1];
          wacc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ws0, ones, wacc[0], 0, 0, 0);
          wacc[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ws1, ones, wacc[1], 0, 0, 0);
        }
      };
      // group 0 has landed when at most group 1's loads are outstanding
      IGR_WAIT(G, 0);
      __builtin_amdgcn_s_barrier();
      IGR_STAMP(1)
#pragma unroll
      for (int t = 0; t < TN; t++) w0[t] = *(const v4i *)(igr_lds + w_lane + t * 1024);
#pragma unroll
      for (int s = 0; s < 4; s++) af[s] = *(const v4i *)(igr_lds + a_lane[0] + a_imm(s, 0));
      int ab = 0, ws = 0;
#pragma unroll 1
      for (int grp = 0; grp < NG; grp++) {
        step(std::integral_constant<int, 0>{}, w0, w1, grp, ab, ws);
        step(std::integral_constant<int, 1>{}, w1, w0, grp, ab, ws);
        step(std::integral_constant<int, 2>{}, w0, w1, grp, ab, ws);
#pragma unroll
        for (int t = 0; t < TN; t++) w0[t] = w1[t];
        ab = ab == 2 ? 0 : ab + 1;
        ws = 1 - ws;
      }
    };
    if (first) main_loop(std::true_type{});
    else main_loop(std::false_type{});
    IGR_STAMP(2)

    if (first) {
      // weight sums -> LDS -> the channel table of the epilogue, exactly as in igemm_ring_kernel
      if (l16 == 0) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int r = 0; r < 4; r++) wsum[wave_n * WNC + 16 * (2 * wave_m + i) + 4 * lgrp + r] = wacc[i][r];
      }
      __syncthreads();
      int tid_o = tid;
      asm volatile("" : "+v"(tid_o));  // (opaque, as in pixel_setup)
      for (int c = tid_o; c < BN; c += IGP_THREADS) {
        const int n = n0 + c;
        const int cc = c % WNC;
        const int row = (c / WNC) * WNC + 16 * ((cc & 15) >> 2) + 4 * (cc >> 4) + (cc & 3);
        int corr = 128 * wsum[row];
        bn_t kv = 0, lv = 0;
        if (n < g.N) {
          if (g.bias) corr += (int)g.bias[n];
          if (MODE == EPI_BN) {
            kv = e.k[n];
            lv = e.lambda[n];
          }
        }
        if (MODE == EPI_BN) {
#if PULPNN_BN_BITS == 64
          cadd[c] = (bn_t)((unsigned long long)kv * (unsigned long long)(long long)corr + (unsigned long long)lv);
#else
          cadd[c] = (bn_t)((unsigned)kv * (unsigned)corr + (unsigned)lv);
#endif
          cmul[c] = kv;
        } else if (MODE == EPI_MULT) {
          cadd[c] = (bn_t)(int)((unsigned)e.mult * (unsigned)corr);
        } else {
          cadd[c] = (bn_t)corr;
        }
      }
      first = false;
      __syncthreads();
    }
    // the next tile's first two groups travel during the epilogue (the last barrier of the loop was passed with
    // every wave's last fragments in registers, and the loop's last request was out of range)
    const int next = tile + gridDim.x;
    if (next < g.tiles_total) {
      pixel_setup(tile_m_of(next));
      first_loads();
    }

    // ---- epilogue: acc[t][s][r] = channel cb + 4*t + r of tile row 2*wave_m + s/4, column 16*(s%4) + l16 ----
    if (!(ABL & 8) || g.M < 0) {
      int lane_o = lane;
      asm volatile("" : "+v"(lane_o));  // (opaque, as in pixel_setup)
      const int l16e = lane_o & 15;
      const int cb = wave_n * WNC + (lane_o >> 4) * 16;
      // (the table offset of this lane is made opaque: the 32 table addresses it leads to are then one register plus
      // immediates, computed here; known to be loop-invariant they are computed before the tile loop, each in a
      // register of its own, and spilled)
      int cbo = cb;
      asm volatile("" : "+v"(cbo));
      unsigned packed[TM][TN];
      auto requantise = [&](auto form_tag) {
        constexpr int FORM = decltype(form_tag)::value;
#pragma unroll
        for (int t = 0; t < TN; t++) {
          bn_t kk[4], ll[4];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            ll[r] = cadd[cbo + 4 * t + r];
            kk[r] = MODE == EPI_BN ? cmul[cbo + 4 * t + r] : (bn_t)0;
          }
#pragma unroll
          for (int s = 0; s < TM; s++) packed[s][t] = igr_requant4<MODE, FORM>(acc[t][s], kk, ll, e);
        }
      };
#if PULPNN_BN_BITS == 64
      if constexpr (MODE == EPI_BN) {
        bool ks = true;
#pragma unroll
        for (int c = 0; c < 16; c++) ks = ks && bn_k_small(cmul[cbo + c]);
        const bool small = __all(ks);  // wave-uniform
        if (small && e.shift >= 32) requantise(std::integral_constant<int, 0>{});
        else if (small) requantise(std::integral_constant<int, 1>{});
        else requantise(std::integral_constant<int, 2>{});
      } else {
        requantise(std::integral_constant<int, 0>{});
      }
#else
      requantise(std::integral_constant<int, 0>{});
#endif
      // the next tile's first group is waited for before the stores go out (one in-order counter for both)
      IGR_WAIT(G, 0);
      auto put = [&](auto nt) {
        constexpr bool NT = decltype(nt)::value;
#pragma unroll
        for (int s = 0; s < TM; s++) {
          const int oy = cur_oy0 + 2 * wave_m + s / 4, ox = 16 * (s % 4) + l16e;
          if (oy < g.Ho && ox < g.Wo && cur_img < g.batch && n0 + cb < g.N) {
            const int m = cur_img * g.HoWo + oy * g.Wo + ox;  // < M
            store16<NT>((uint8_t *)g.out + (long long)m * g.N + n0 + cb,
                        (v4i){(int)packed[s][0], (int)packed[s][1], (int)packed[s][2], (int)packed[s][3]});
          }
        }
      };
      if constexpr ((ABL & 16) != 0) {
        unsigned x = 0;
#pragma unroll
        for (int s = 0; s < TM; s++)
#pragma unroll
          for (int t = 0; t < TN; t++) x ^= packed[s][t];
        if (x == 0x12345678u && g.M < 0) *(unsigned *)g.out = x;
      } else {
        if (g.nt) put(std::true_type{});
        else put(std::false_type{});
      }
    }
    IGR_STAMP(3)
#ifdef IGR_TRACE
    round++;
#endif
  }
}
