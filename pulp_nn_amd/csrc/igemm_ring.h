// Implicit-GEMM kernel for large standard convolutions (and any GEMM of the same shape) whose input
// channels are a multiple of 64: the MFMA-bound case of
// 32bit/src/pulp_nn_conv_Ho_parallel.c:76-183 + pulp_nn_matmul.c:53-216.
//
// Same arithmetic as igemm_kernel (activations as a ^ 0x80, 128 * sum_k w added back, identical
// requantisation); what differs is how the operands reach the matrix cores and how the work is laid out in time:
//   * the operands travel HBM/L2 -> LDS with buffer loads that write LDS directly
//     (buffer_load_dwordx4 ... lds): no staging registers, no LDS store instructions.  A wave's load writes
//     1 KB of consecutive LDS (lane l at 16*l), so the XOR swizzle that makes the fragment reads conflict-free
//     is applied to the global address each lane fetches instead of to the LDS address it writes.  An
//     out-of-image tap is an out-of-range buffer load, which writes zeros (0x80 after the xor, which is applied
//     to the activation fragments after they are read from LDS);
//   * the weight sums come from the matrix core as well: a weight fragment times a matrix of ones gives the
//     sums of its 16 rows.  Each wave does that for two of its four fragments; the two waves that share the
//     fragments (same channels, other pixel half) split them between them (v_dot4 on the fragments costs
//     several times the issue slots and holds up the MFMAs behind it);
//   * persistent workgroups: a workgroup walks over pixel tiles of one channel range.  It computes the weight
//     sums while it multiplies its first tile and keeps them (2 MFMAs in 34 saved on the other tiles), folds
//     them, the bias and the requantisation parameters into one table per channel once, and requests the
//     first sub-slices of its next tile before the epilogue of the current one;
//   * K is taken in sub-slices of 64 bytes through a ring of NS LDS stages: the loads of sub-slice j + NS are
//     issued when sub-slice j's fragments have left LDS, and they have NS - 1 iterations to land;
//   * the fragments of sub-slice j + 1 are read from LDS while sub-slice j is multiplied: an activation
//     fragment's registers are refilled as soon as its four MFMAs are issued, the weight fragments have two
//     register sets.  No MFMA waits for an LDS read issued just before it; one barrier per sub-slice;
//   * the epilogue is straight-line code: which form of the requantisation applies (multiplier width, shift
//     range) is decided once per workgroup, not per group of four outputs, and the per-channel additive terms
//     are folded into one constant: k * (acc + corr) + lambda = k * acc + (k * corr + lambda), exact in the
//     wrapping arithmetic of the reference's types.
// Tile: 256 pixels x 64*WN channels, wave tiles of 128 x 64 (32 MFMAs per 12 fragment reads), 2*WN waves.
//   WN = 4: one workgroup of eight waves per compute unit, 256 x 256 tiles (fewest bytes from L2 per multiply);
//   WN = 2: two workgroups of four waves per compute unit on 256 x 128 tiles, which run independently of
//           each other (one's epilogue overlaps the other's main loop) at 1.5 x the bytes from L2.
#pragma once
#include "igemm.h"

#define IGR_BM 256
#define IGR_A_BYTES (IGR_BM * 64)

template <int WN>
struct IgrShape {
  static constexpr int NWAVES = 2 * WN;
  static constexpr int THREADS = 64 * NWAVES;
  static constexpr int BN = 64 * WN;
  static constexpr int NS = WN == 2 ? 3 : 4;           // LDS stages
  static constexpr bool PAIR = NS == 4;                // sub-slices are requested two at a time
  static constexpr int STAGE = IGR_A_BYTES + BN * 64;  // bytes per stage
  static constexpr int GA = 16 / NWAVES;               // activation loads per wave and sub-slice (16 rows each)
  static constexpr int GW = 2;                         // weight loads per wave and sub-slice
  static constexpr int G = GA + GW;
  // dynamic LDS: the ring, then per channel: weight sum, folded additive constant, multiplier
  static int lds_bytes() { return NS * STAGE + BN * (4 + 2 * (int)sizeof(bn_t)); }
};

// s_waitcnt immediate: at most n vector-memory operations outstanding; LGK: also wait for all LDS reads
#define IGR_WAIT(n, LGK) __builtin_amdgcn_s_waitcnt((((n) & 15) | (((n) >> 4) << 14) | 0x70 | ((LGK) ? 0 : 0xF00)))

// IGR_TRACE (tools only): thread 0 of every workgroup writes, per tile, the 100 MHz wall clock and the shader
// cycle counter at the start of the tile, when its first sub-slice is in LDS, at the end of the main loop and
// at the end of the epilogue, to igr_trace[(workgroup * 8 + tile round) * 8 ...].
#ifdef IGR_TRACE
__device__ long long *igr_trace = nullptr;
#define IGR_STAMP(i)                                                                                 \
  if (igr_trace && tid == 0 && round < 8) {                                                          \
    igr_trace[((long long)blockIdx.x * 8 + round) * 8 + 2 * (i)] = wall_clock64();                   \
    igr_trace[((long long)blockIdx.x * 8 + round) * 8 + 2 * (i) + 1] = __builtin_readcyclecounter(); \
  }
#else
#define IGR_STAMP(i)
#endif

// Requantisation of four accumulators (consecutive channels of one pixel) with the folded per-channel constants:
// ll = k * corr + lambda (batch-norm branch), mult * corr (scalar multiplier) or corr (shift only), see the
// kernels' channel tables.  FORM (batch-norm branch, 64-bit build): 0 = multipliers fit 32 bits and shift >= 32
// (the result is the high dword of k * acc + l, shifted), 1 = multipliers fit 32 bits (funnel shift of the two
// dwords), 2 = general 64-bit arithmetic.  Other branches and the 32-bit build have one form.
template <int MODE, int FORM>
__device__ __forceinline__ unsigned igr_requant4(const v4i &a, const bn_t (&kk)[4], const bn_t (&ll)[4], const EpiArgs &e)
{
  int x[4];
  if constexpr (MODE == EPI_BN) {
#if PULPNN_BN_BITS == 64
    if constexpr (FORM == 0) {
#pragma unroll
      for (int r = 0; r < 4; r++) x[r] = (int)(((long long)(int)kk[r] * (long long)a[r] + ll[r]) >> 32);
      return ashr_sat_pack4(x[0], x[1], x[2], x[3], e.shift - 32);
    } else if constexpr (FORM == 1) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const long long v = (long long)(int)kk[r] * (long long)a[r] + ll[r];
        x[r] = (int)__builtin_amdgcn_alignbit((unsigned)(v >> 32), (unsigned)v, e.shift);
      }
      return ashr_sat_pack4(x[0], x[1], x[2], x[3], 0);
    } else {
      unsigned p = 0;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const unsigned long long v = (unsigned long long)kk[r] * (unsigned long long)(long long)a[r] + (unsigned long long)ll[r];
        p |= (unsigned)clipu8((int)(unsigned)(unsigned long long)((long long)v >> e.shift)) << (8 * r);
      }
      return p;
    }
#else
#pragma unroll
    for (int r = 0; r < 4; r++) x[r] = (int)((unsigned)kk[r] * (unsigned)a[r] + (unsigned)ll[r]);
    return ashr_sat_pack4(x[0], x[1], x[2], x[3], e.shift);
#endif
  } else if constexpr (MODE == EPI_MULT) {
    // (int16_t)((mult * (acc + corr)) >> shift), then clamp
#pragma unroll
    for (int r = 0; r < 4; r++) x[r] = (int)(short)((int)((unsigned)e.mult * (unsigned)a[r] + (unsigned)ll[r]) >> e.shift);
    return ashr_sat_pack4(x[0], x[1], x[2], x[3], 0);
  } else {
#pragma unroll
    for (int r = 0; r < 4; r++) x[r] = (a[r] + (int)ll[r]) >> e.shift;
    return ashr_sat_pack4(x[0], x[1], x[2], x[3], 0);
  }
}

// ABL (tools only, wrong results): 1 = no loads after a tile's first sub-slices, 2 = one MFMA per
// sub-slice instead of 32, 4 = no fragment reads in the loop, 8 = no epilogue, 16 = epilogue without its stores.
template <int MODE, int WN, int ABL = 0>
__global__ __launch_bounds__(IgrShape<WN>::THREADS, WN == 2 ? 2 : 1) void igemm_ring_kernel(ConvGeom g, EpiArgs e)
{
  typedef IgrShape<WN> S;
  constexpr int TM = 8, TN = 4, WM = 128, WNC = 64, BM = IGR_BM, BN = S::BN, NS = S::NS, G = S::G;
  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char igr_lds[];
  int *wsum = (int *)(igr_lds + NS * S::STAGE);  // weight sums by LDS row
  bn_t *cadd = (bn_t *)(wsum + BN);              // per channel: additive constant of the epilogue
  bn_t *cmul = cadd + BN;                        // per channel: multiplier (batch-norm branch)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave & 1, wave_n = wave >> 1;
  const int l16 = lane & 15, lgrp = lane >> 4;

  // Tiles of this workgroup: t, t + gridDim.x, ... (the grid is a multiple of 8 * tiles_n, so all of them have
  // the same channel offset).  Workgroups are dealt round-robin to the 8 XCDs; t gives each XCD a contiguous
  // range of tiles, so that the channel ranges of a pixel tile and its neighbours (shared halo rows) meet in
  // one L2.
  // (No early exit for a workgroup without a tile: the host launches no more workgroups than tiles, and one
  // without a tile would request zeros and skip the loop.  An exit here makes the compiler treat the scalar
  // state of the loop as divergent.)
  int tile = (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3);
  auto tile_m_of = [&](int t) { return (int)fastdiv((unsigned)t, g.d_tiles_n); };
  const int n0 = (tile - tile_m_of(tile) * g.tiles_n) * BN;

  const unsigned OOB = 0x80000000u;  // offsets stay below 2^31 (checked by the host), so this bit puts a load out of range
  const unsigned shift = (unsigned)((g.pt * g.W + g.pl) * g.Ci);
  const unsigned batch = (unsigned)g.batch;
  const __amdgpu_buffer_rsrc_t rsrc_a =
      __builtin_amdgcn_make_buffer_rsrc((void *)(g.in - shift), 0, shift + batch * (unsigned)g.in_img, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)g.w, 0, (unsigned)g.N * (unsigned)g.K, 0x00020000);

  // ---- what this lane fetches ------------------------------------------------------------------
  // A load instruction fills 16 rows of a stage (64 bytes each): lane l writes slot l%4 of row l/4 of
  // the block, which has to hold K chunk (l%4) ^ ((row/2)%4).  Wave w loads activation blocks
  // GA*w .. GA*w + GA-1 and weight blocks 2w, 2w+1.
  unsigned poff[S::GA], pinv[S::GA], woff[S::GW];
#pragma unroll
  for (int j = 0; j < S::GW; j++) {
    const int row = 16 * (S::GW * wave + j) + (lane >> 2);
    const unsigned chunk = (unsigned)((lane & 3) ^ ((row >> 1) & 3));
    // weight rows sit in LDS in fragment order (see igemm_kernel): LDS row p holds channel
    // (p/64)*64 + ((p%16)/4)*16 + 4*((p%64)/16) + p%4
    const int pp = row % WNC, t = pp >> 4, r16 = pp & 15;
    const int n = n0 + (row / WNC) * WNC + (r16 >> 2) * (4 * TN) + 4 * t + (r16 & 3);
    woff[j] = n < g.N ? (unsigned)n * (unsigned)g.K + 16u * chunk : OOB;
  }
  auto pixel_setup = [&](int m0) {
#pragma unroll
    for (int j = 0; j < S::GA; j++) {
      const int row = 16 * (S::GA * wave + j) + (lane >> 2);
      const unsigned chunk = (unsigned)((lane & 3) ^ ((row >> 1) & 3));
      const int m = m0 + row;
      poff[j] = OOB;
      pinv[j] = 0;
      if (m < g.M) {
        const int b = (int)fastdiv((unsigned)m, g.d_howo), rem = m - b * g.HoWo;
        const int oy = (int)fastdiv((unsigned)rem, g.d_wo), ox = rem - oy * g.Wo;
        poff[j] = (unsigned)b * (unsigned)g.in_img + (unsigned)((oy * g.sy * g.W + ox * g.sx) * g.Ci) + 16u * chunk;
        // taps outside the image: filter rows fy with iy = oy*sy - pt + fy outside [0, H) and columns fx
        // likewise; one bit per tap t = fy*kx + fx (the host checks ky*kx <= 32)
        const int iy0 = oy * g.sy - g.pt, ix0 = ox * g.sx - g.pl;
        const int fx_lo = max(-ix0, 0), fx_hi = min(g.W - ix0, g.kx);   // valid columns: fx_lo <= fx < fx_hi
        const unsigned cols = fx_hi > fx_lo ? ((fx_hi >= 32 ? 0u : 1u << fx_hi) - (1u << fx_lo)) : 0u;
        unsigned valid = 0;
        for (int fy_ = 0; fy_ < g.ky; fy_++)
          valid |= ((unsigned)(iy0 + fy_) < (unsigned)g.H ? cols : 0u) << (fy_ * g.kx);
        pinv[j] = ~valid;
      }
    }
  };

  // The next sub-slice to request.  Its tap and first channel are computed from the counter (scalar
  // multiply-high divisions by launch constants): state carried through selects or branches ends up in
  // vector registers, and the loads' scalar offset would then be read back lane by lane.
  int u_slice = 0;
  const int KT = g.K / 64;
  auto slice_offset = [&](int slice, int &tap_out) {
    const unsigned tap = fastdiv((unsigned)slice, g.d_cpt);    // sub-slices per tap: Ci / 64
    const unsigned ci = ((unsigned)slice - tap * (unsigned)g.cpt) * 64u;
    const unsigned fy = fastdiv(tap, g.d_kx), fx = tap - fy * (unsigned)g.kx;
    tap_out = __builtin_amdgcn_readfirstlane((int)tap);
    return __builtin_amdgcn_readfirstlane((int)((fy * (unsigned)g.W + fx) * (unsigned)g.Ci + ci));
  };
  // NSUB sub-slices (1 or 2) into the stages stage, stage + 1: with two, the loads of a 16-row block for the
  // first and the second sub-slice follow each other.  With Ci a multiple of 128 those are the two halves of the
  // same 128-byte lines; issued an iteration apart, each half is a request of its own to L2 (twice the requests
  // for the same bytes), back to back the second one finds the line in the vector cache.
  auto dma = [&](auto nsub_tag, int stage, unsigned dead0, unsigned dead1) {
    constexpr int NSUB = decltype(nsub_tag)::value;
    int tap[2], soff_a[2], soff_w[2];
    unsigned dead[2] = {dead0, dead1};
#pragma unroll
    for (int h = 0; h < NSUB; h++) {
      soff_a[h] = slice_offset(u_slice + h, tap[h]);
      soff_w[h] = (u_slice + h) * 64;
    }
    unsigned char *a_dst = igr_lds + stage * S::STAGE + wave * (1024 * S::GA);
    unsigned char *w_dst = igr_lds + stage * S::STAGE + IGR_A_BYTES + wave * (1024 * S::GW);
#pragma unroll
    for (int j = 0; j < S::GA; j++)
#pragma unroll
      for (int h = 0; h < NSUB; h++) {
        const unsigned oob = ((unsigned)__builtin_amdgcn_sbfe((int)pinv[j], tap[h], 1) & OOB) | dead[h];
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)(a_dst + h * S::STAGE + 1024 * j), 16, (int)(poff[j] | oob),
                                                 soff_a[h], 0, 0);
      }
#pragma unroll
    for (int j = 0; j < S::GW; j++)
#pragma unroll
      for (int h = 0; h < NSUB; h++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr_t)(w_dst + h * S::STAGE + 1024 * j), 16, (int)(woff[j] | dead[h]),
                                                 soff_w[h], 0, 0);
    u_slice += NSUB;
  };
  auto first_loads = [&]() {
    u_slice = 0;  // (the host guarantees KT >= NS)
    if constexpr (S::PAIR) {
      dma(std::integral_constant<int, 2>{}, 0, 0u, 0u);
      dma(std::integral_constant<int, 2>{}, 2, 0u, 0u);
    } else {
#pragma unroll
      for (int j = 0; j < NS; j++) dma(std::integral_constant<int, 1>{}, j, 0u, 0u);
    }
  };

  // fragment addresses of this lane: row r of a stage at 64*r, chunk c of it in slot c ^ ((r/2)%4)
  const int swz = (lgrp ^ ((l16 >> 1) & 3)) << 4;
  const int a_lane = (wave_m * WM + l16) * 64 + swz;
  const int w_lane = IGR_A_BYTES + (wave_n * WNC + l16) * 64 + swz;

  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
  v4i acc[TN][TM];
  v4i wacc[2];

  pixel_setup(tile_m_of(tile) * BM);
  first_loads();

  bool first = true;
  [[maybe_unused]] int round = 0;
#pragma unroll 1
  for (; tile < g.tiles_total; tile += gridDim.x) {
    const int m0 = tile_m_of(tile) * BM;
    IGR_STAMP(0)
#pragma unroll
    for (int t = 0; t < TN; t++)
#pragma unroll
      for (int s = 0; s < TM; s++) acc[t][s] = (v4i){0, 0, 0, 0};
    wacc[0] = wacc[1] = (v4i){0, 0, 0, 0};

    // The loop over the sub-slices of one tile.  WS: also accumulate the weight sums.
    auto main_loop = [&](auto ws_tag) {
      constexpr bool WS = decltype(ws_tag)::value;
      // Fragment registers: one set of activation fragments, refilled in place (fragment s of the next
      // sub-slice is requested as soon as the MFMAs of fragment s of this one are issued, a whole iteration
      // before it is needed), and two sets of weight fragments.
      v4i af[TM], w0[TN], w1[TN];
      // One iteration: the loads of sub-slice kt + 1 have landed (those of the NS - 2 after it may still be in
      // flight) and this wave's fragments of sub-slice kt are in registers; after the barrier that holds for
      // every wave, so the stage of sub-slice kt can take sub-slice kt + NS and the next stage can be read.
      // (The last iteration reads a stage that holds nothing of this tile; those fragments are never used.)
      auto step = [&](auto odd_tag, v4i (&wc)[TN], v4i (&wn)[TN], int kt, int stage) {
        constexpr bool ODD = decltype(odd_tag)::value;
        // (no branch around the loads: past the end of K they are requested out of range, which costs no
        // memory traffic, keeps the count of loads in flight the same in every iteration, and leaves the
        // iteration one basic block, so that the loads can be placed between the MFMAs)
        if constexpr (S::PAIR) {
          // four stages, loads in pairs: behind the barrier of an odd iteration the stages of sub-slices kt - 1
          // and kt are free and take kt + 3 and kt + 4.  An even iteration needs the pair (kt, kt + 1), with
          // the pair after it in flight; an odd one needs the pair (kt + 1, kt + 2), the youngest.
          if constexpr (ODD) IGR_WAIT(0, 1);
          else IGR_WAIT(2 * G, 1);
          __builtin_amdgcn_s_barrier();
          if (ODD && !(ABL & 1))
            dma(std::integral_constant<int, 2>{}, stage == 0 ? NS - 1 : stage - 1, kt + 3 < KT ? 0u : OOB, kt + 4 < KT ? 0u : OOB);
        } else {
          IGR_WAIT((NS - 2) * G, 1);
          __builtin_amdgcn_s_barrier();
          if (!(ABL & 1)) dma(std::integral_constant<int, 1>{}, stage, kt + NS < KT ? 0u : OOB, 0u);
        }
        const unsigned char *nb = igr_lds + (stage == NS - 1 ? 0 : stage + 1) * S::STAGE;
#pragma unroll
        for (int s = 0; s < TM; s++) {
          const v4i a = af[s] ^ (int)0x80808080;
#pragma unroll
          for (int t = 0; t < TN; t++)
            if (!(ABL & 2) || (s == 0 && t == 0)) acc[t][s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wc[t], a, acc[t][s], 0, 0, 0);
          if (!(ABL & 4)) {
            af[s] = *(const v4i *)(nb + a_lane + s * 1024);
            if (s < TN) wn[s] = *(const v4i *)(nb + w_lane + s * 1024);
          } else if (s < TN) {
            wn[s] = wc[s];
          }
        }
        if constexpr (WS) {
          // (a select, not a branch: wave_m is uniform, and a branch here splits the loop body)
          const v4i ws0 = wave_m ? wc[2] : wc[0], ws1 = wave_m ? wc[3] : wc[1];
          wacc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ws0, ones, wacc[0], 0, 0, 0);
          wacc[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ws1, ones, wacc[1], 0, 0, 0);
        }
        // Keep the instructions where they are written.  Left to itself the scheduler puts all 32 xors and the
        // loads' address arithmetic in front of the first MFMA (the matrix cores idle meanwhile, for all waves
        // leave the barrier together) and sinks reads to the end of the iteration, where the next one waits
        // for them.  0x002: vector ALU, 0x008: MFMA, 0x020: vector memory read, 0x100: LDS read
#define IGR_GROUP(nread, nload)                          \
  __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);     \
  __builtin_amdgcn_sched_group_barrier(0x020, nload, 0); \
  __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);     \
  __builtin_amdgcn_sched_group_barrier(0x100, nread, 0);
        if constexpr (ABL == 0) {
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
          constexpr int NL = S::PAIR ? (ODD ? 2 * G : 0) : G;  // loads of this iteration, spread over four groups
          IGR_GROUP(2, NL / 4) IGR_GROUP(2, NL / 4) IGR_GROUP(2, NL / 4) IGR_GROUP(2, NL - 3 * (NL / 4)) IGR_GROUP(1, 0) IGR_GROUP(1, 0) IGR_GROUP(1, 0)
          __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
#undef IGR_GROUP
      };
      // sub-slice 0: its loads are the oldest of the NS groups in flight (in pairs: the first of two pairs)
      IGR_WAIT(S::PAIR ? 2 * G : (NS - 1) * G, 0);
      __builtin_amdgcn_s_barrier();
      IGR_STAMP(1)
#pragma unroll
      for (int t = 0; t < TN; t++) w0[t] = *(const v4i *)(igr_lds + w_lane + t * 1024);
#pragma unroll
      for (int s = 0; s < TM; s++) af[s] = *(const v4i *)(igr_lds + a_lane + s * 1024);
      int stage = 0;
#pragma unroll 1
      for (int kt = 0; kt < KT; kt += 2) {
        step(std::false_type{}, w0, w1, kt, stage);
        stage = stage == NS - 1 ? 0 : stage + 1;
        if (kt + 1 < KT) step(std::true_type{}, w1, w0, kt + 1, stage);
        stage = stage == NS - 1 ? 0 : stage + 1;
      }
    };
    if (first) main_loop(std::true_type{});
    else main_loop(std::false_type{});
    IGR_STAMP(2)

    if (first) {
      // ---- per-row weight sums -> LDS (indexed by LDS row) -------------------------------------------
      // wacc[i][r] of a lane = sum of LDS weight row 16*t + 4*(lane/16) + r of this wave's channels, t = 2*wave_m + i
      if (l16 == 0) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int r = 0; r < 4; r++) wsum[wave_n * WNC + 16 * (2 * wave_m + i) + 4 * lgrp + r] = wacc[i][r];
      }
      __syncthreads();
      // ---- the channel table of the epilogue: acc + corr with corr = bias + 128 * weight sum, folded into
      // the requantisation: k * (acc + corr) + lambda = k * acc + (k * corr + lambda) (batch-norm branch, mod
      // 2^32 or 2^64 as the reference's types wrap), mult * (acc + corr) = mult * acc + mult * corr (mod 2^32).
      for (int c = tid; c < BN; c += S::THREADS) {
        const int n = n0 + c;
        // channel c of the tile sits in LDS weight row (c/64)*64 + 16*((c%16)/4) + 4*((c%64)/16) + c%4
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
    // The next tile's first sub-slices travel during the epilogue.  (Every wave had its last fragments of this
    // tile in registers before the last barrier of the loop, so the stages are free.)
    const int next = tile + gridDim.x;
    if (next < g.tiles_total) {
      pixel_setup(tile_m_of(next) * BM);
      first_loads();
    }

    // ---- epilogue: acc[t][s][r] = channel cb + 4*t + r of pixel m0 + wave_m*128 + 16*s + l16 -----------
    // Four channels (one t) at a time, so that only their constants are in registers next to the accumulators.
    if (!(ABL & 8) || g.M < 0) {
      const int cb = wave_n * WNC + lgrp * 16;
      unsigned packed[TM][TN];
      // FORM: see igr_requant4
      auto requantise = [&](auto form_tag) {
        constexpr int FORM = decltype(form_tag)::value;
#pragma unroll
        for (int t = 0; t < TN; t++) {
          bn_t kk[4], ll[4];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            ll[r] = cadd[cb + 4 * t + r];
            kk[r] = MODE == EPI_BN ? cmul[cb + 4 * t + r] : (bn_t)0;
          }
#pragma unroll
          for (int s = 0; s < TM; s++) packed[s][t] = igr_requant4<MODE, FORM>(acc[t][s], kk, ll, e);
        }
      };
#if PULPNN_BN_BITS == 64
      if constexpr (MODE == EPI_BN) {
        bool ks = true;
#pragma unroll
        for (int c = 0; c < 16; c++) ks = ks && bn_k_small(cmul[cb + c]);
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
      // The next tile's first sub-slice is waited for before the stores go out: behind them the same wait would
      // also wait for the stores (one in-order counter for loads and stores).
      IGR_WAIT(S::PAIR ? 2 * G : (NS - 1) * G, 0);
      auto put = [&](auto nt) {
        constexpr bool NT = decltype(nt)::value;
#pragma unroll
        for (int s = 0; s < TM; s++) {
          const int m = m0 + wave_m * WM + 16 * s + l16;
          if (m < g.M && n0 + cb < g.N)
            store16<NT>((uint8_t *)g.out + (long long)m * g.N + n0 + cb,
                        (v4i){(int)packed[s][0], (int)packed[s][1], (int)packed[s][2], (int)packed[s][3]});
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
