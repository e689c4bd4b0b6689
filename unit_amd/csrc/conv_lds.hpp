// Implicit-GEMM int8 convolution (NCHW16c data, prepared weights) whose operand tiles are shared by the
// waves of a workgroup through LDS and arrive there straight from global memory
// (global_load_lds_dwordx4, no VGPR round trip) through a ring of NST (3 to 6) stage buffers.
//
// X operand = weights: the prepared buffer already holds MFMA fragments, 1 KiB per (32-channel block,
// k-step), so a wave-level direct load moves one fragment and a lane reads it back at lane * 16.
// Y operand = pixels, gathered on the fly: a k-step is two taps (ci, kh, kw) of 16 input channels, and
// in NCHW16c the 16 channels of a pixel and tap are 16 contiguous bytes, consecutive pixels of an image
// row consecutive in memory.  One direct load moves (64 pixel rows) x (one tap): lane i fetches the 16
// bytes of row i -- coalesced along the image row -- and they land in LDS as [tap slot][row][16 bytes],
// which is also the conflict-free order for the fragment reads (lanes 0-31 one tap, 32-63 the next, 32
// consecutive rows each).  Zero padding is the hardware's: the pixel loads are raw buffer loads over the data
// tensor, a lane whose tap falls outside the image is given an offset past the tensor, and an out-of-range lane
// of a buffer load stores zeros -- no masks or selects on the data path.  The lane's offset of each window
// position is computed once per workgroup into an LDS table; per load the wave reads one entry and adds the
// channel block's offset as the load's scalar offset.  The u8 -> s8 shift is one XOR per fragment dword after
// the fragment read, its correction 128 * sum(w) comes precomputed with the prepared weights.
//
// Pipeline.  Stage kt (KS k-steps) is computed from buffer kt % NST while the direct loads of stage
// kt + NST - 1 are issued into the buffer that stage kt - 1 freed, spread over the stage's MFMAs, and the
// stages between are landing: NST - 1 stages of loads are in flight throughout.  Fragments are double-buffered in registers
// across k-steps and across the stage boundary; one workgroup barrier per stage, placed before the
// stage's last k-step.
//
// KG k-groups of WX x WY waves share the output tile, each on its own share of the k-steps with its own
// ring; partial tiles meet in LDS and all waves share the write-back.
#pragma once
#include "conv_direct.hpp"
#include "mma_dma.hpp"

namespace unit {

template <int TX_, int TY_, int WX_, int WY_, int KG_, int KS_, int NST_ = 3>
struct LdsShape {
  static constexpr int TX = TX_, TY = TY_, WX = WX_, WY = WY_, KG = KG_, KS = KS_, NST = NST_;
  static constexpr int BX = 32 * TX * WX, BY = 32 * TY * WY;  // channels x pixels per workgroup
  static constexpr int NWG = WX * WY, NW = NWG * KG, NT = 64 * NW;
  static constexpr int XB = BX / 32, YB = BY / 32, RG = BY / 64;  // fragment blocks; 64-row groups of pixels
  static constexpr int NX = KS * XB, NY = 2 * KS * RG;            // direct loads (1 KiB each) per stage and k-group
  static constexpr int LX = NX / NWG, LY = NY / NWG, LW = LX + LY;  // per wave
  static constexpr int XPART = NX * 1024, STAGE = XPART + NY * 1024, RING = NST * STAGE;
  static constexpr int NM = TX * TY, NF = TX + TY;
  static constexpr int LPK = (LW + KS - 1) / KS;                     // direct loads issued per k-step
  static constexpr int NBLK = XB * YB, NBW = (NBLK + NW - 1) / NW;  // 32 x 32 blocks of the tile; per wave in the write-back
  static constexpr int kScratch = 32 * 144 + 128;  // per wave: transpose area + 32 addends
  // the write-back reuses the rings: parked partial tiles (KG > 1), then the waves' transpose areas
  static constexpr int kPark = KG > 1 ? KG * BX * BY * 4 : 0;
  static constexpr int kBack = kPark + NW * kScratch;
  static constexpr int kMain = KG * RING > kBack ? KG * RING : kBack;  // the tap table follows
  static_assert(BY % 64 == 0, "pixel rows come in groups of 64 (one direct load)");
  static_assert(NX % NWG == 0 && NY % NWG == 0, "direct loads split evenly over the waves of a k-group");
  static_assert(NWG % RG == 0, "a wave gathers rows of one 64-pixel group only");
  static_assert(KS % 2 == 0, "fragment double buffering needs an even number of k-steps per stage");
  static_assert(NM >= NF && NM >= LPK, "a k-step has too few MFMAs to carry its fragment reads and direct loads");
  static_assert(NT <= 1024 && NST >= 3 && NST <= 6, "at most 16 waves; ring of 3 to 6 buffers");
};

// The direct loads are written out as instructions, so that the compiler's counter bookkeeping does not see
// them (it would make LDS reads that follow a direct load wait for all of them); the kernel's own vmcnt waits
// order them.  Weight fragments: scalar base + the lane's 16-byte offset.  Pixel rows: a raw buffer load, whose
// out-of-range lanes store zeros into LDS -- the hardware's own zero padding.
// The statements write m0 without naming it as a clobber: the compiler reserves m0 (it sets it right before each
// instruction of its own that reads it and keeps no value in it across statements) and rejects it in a clobber list.
__device__ __forceinline__ void dma_global_16(u32 lds_addr, u32 voff, const void *sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void dma_buffer_16(u32 lds_addr, u32 voff, v4i rsrc, u32 soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}

// fp16 (Op = OpF16): a pixel and tap are 32 bytes, one k-step; the two 16-byte halves (input channels 0-7 and 8-15) take
// the places of the int8 kernel's two taps of a k-step, so the tiling in bytes is the same.  The prepared fp16 weights
// have no zero region behind them: their fragments come by buffer loads as well, out of range past a k-group's share.
template <class S, bool SHIFT, bool Q8 = false, bool NCHW = false, class Op = OpI8>
__global__ __launch_bounds__(S::NT) void conv_lds(const char *__restrict__ data, const char *__restrict__ wgt,
                                                  const char *__restrict__ zero, typename ConvEpilogue<Op>::Params ep,
                                                  ConvGeom g, GridMap gm, int nsteps) {
  constexpr bool F16 = !Op::kInt;
  constexpr int ESZ = F16 ? 2 : 1;          // bytes per element
  constexpr int SPT = F16 ? 2 : 1;          // 16-byte slots of the pixel tile per tap
  static_assert(!F16 || (!SHIFT && !Q8), "the u8 shift and the requantised output are int8 forms");
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int TX = S::TX, TY = S::TY, KG = S::KG, KS = S::KS, NST = S::NST, LW = S::LW, NM = S::NM, NF = S::NF;
  constexpr int LPK = S::LPK, LX = S::LX, LY = S::LY;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int grp = wave / S::NWG, wg = wave % S::NWG;
  const int wx = wg % S::WX, wy = wg / S::WX;
  const int l32 = lane & 31, half = lane >> 5;

  // k-steps [s0, s1) of this k-group, in stages of KS; every group runs `rounds` stages (one barrier each).  The
  // k-steps of a last stage that lie past s1 are computed on zero weights.
  const int s0 = nsteps * grp / KG, s1 = nsteps * (grp + 1) / KG;
  const int rounds = ((nsteps + KG - 1) / KG + KS - 1) / KS;
  const int nst = (s1 - s0 + KS - 1) / KS;

  int bx, by, split;
  gm.locate(blockIdx.x, bx, by, split);
  const int x0 = bx * S::BX, y0 = by * S::BY;
  char *ring = lds + grp * S::RING;
  const u32 ring_addr = (u32)(uintptr_t)(lptr_t)ring;

  // Position table, per 64-row group of the tile: postab[rg][p][lane] = byte offset in the data tensor of window
  // position p = kh * KW + kw of the row's pixel, channel block 0 -- or an offset past the tensor when that position
  // lies outside the image (or the row is past the last pixel): the buffer load then stores zeros.  Row npos is
  // out of range for every lane (taps past the last one).
  const int npos = g.KH * g.KW;
  constexpr u32 kOutside = 0x80000000u;
  u32 *postab = reinterpret_cast<u32 *>(lds + S::kMain);
  if (wave < S::RG) {
    const int m = y0 + wave * 64 + lane;
    u32 inside = 0;
    int pixoff = 0;
    if (m < g.npix) {
      int n, rem, oh, ow;
      g.by_ohw.divmod(m, n, rem);
      g.by_ow.divmod(rem, oh, ow);
      const int ih0 = oh * g.sh - g.pt, iw0 = ow * g.sw - g.pl;
      pixoff = (int)(n * g.img_bytes) + (ih0 * g.W + iw0) * (16 * ESZ);
      u32 cols = 0, bits = 0;
      for (int kw = 0; kw < g.KW; ++kw) cols |= (u32)((u32)(iw0 + kw * g.dw) < (u32)g.W) << kw;
      for (int kh = 0; kh < g.KH; ++kh)
        if ((u32)(ih0 + kh * g.dh) < (u32)g.H) bits |= cols << (kh * g.KW);
      inside = bits;
    }
    u32 *mine = postab + wave * (npos + 1) * 64 + lane;
    int p = 0;
    for (int kh = 0; kh < g.KH; ++kh)
      for (int kw = 0; kw < g.KW; ++kw, ++p)
        mine[p * 64] = ((inside >> p) & 1u) ? (u32)(pixoff + (kh * g.dh * g.W + kw * g.dw) * (16 * ESZ)) : kOutside;
    mine[npos * 64] = kOutside;
  }

  const int lastkb = (ep.K - 1) >> 5;
  const u32 lane16 = (u32)lane * 16u;
  // raw buffers (base, no stride, size in bytes) over the data tensor and, fp16, over the weight fragments
  auto raw_buffer = [](const char *ptr, u32 bytes) {
    const unsigned long long base = (unsigned long long)ptr;
    v4i r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(u32)base);
    r[1] = __builtin_amdgcn_readfirstlane((int)((u32)(base >> 32) & 0xffffu));
    r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    r[3] = 0x00020000;
    return r;
  };
  const v4i rsrc = raw_buffer(data, (u32)g.N * g.img_bytes);
  const v4i wsrc = raw_buffer(wgt, (u32)(lastkb + 1) * (u32)nsteps * 1024u);

  // ---- this wave's direct loads of a stage, as scalar state that advances from stage to stage (they are issued
  // strictly in stage order): LX weight fragments (KiB q = wg + n * NWG of the stage's X part: k-step q / XB,
  // channel block q % XB), then LY pixel loads (KiB q of the Y part: tap slot q / RG of the stage, row group q % RG)
  const char *xsrc[LX];
  int xs[LX];
#pragma unroll
  for (int n = 0; n < LX; ++n) {
    const int q = wg + n * S::NWG, ks = q / S::XB, xb = q % S::XB;
    int kb = (x0 >> 5) + xb;
    kb = kb < lastkb ? kb : lastkb;
    xs[n] = s0 + ks;
    xsrc[n] = wgt + ((size_t)kb * nsteps + xs[n]) * 1024;
  }
  const int rg = wg % S::RG;
  const u32 chw16 = (u32)g.H * (u32)g.W * (16u * ESZ);  // bytes from one 16-channel block of an image to the next
  constexpr int TPS = 2 * KS / SPT;                      // taps per stage
  const int step_ci = g.by_kh.div(g.by_kw.div(TPS)), step_pos = TPS - step_ci * npos;  // = ci blocks + positions
  // the taps of this k-group end here: past it the pixel loads fetch zeros (int8: the weights there are zero and any
  // finite data would do; fp16: zero weights times data that may hold infinities must not be formed)
  const int tap_end = F16 ? (s1 < g.ntaps ? s1 : g.ntaps) : g.ntaps;
  int ytap[LY], ypos[LY];
  u32 yci[LY];
#pragma unroll
  for (int n = 0; n < LY; ++n) {
    const int slot = 2 * s0 + (wg + n * S::NWG) / S::RG;  // 16-byte slot of the pixel tile, counted over the whole reduction
    const int t = slot / SPT;
    const int ci = g.by_kh.div(g.by_kw.div(t));
    ytap[n] = t;
    ypos[n] = t - ci * npos;
    yci[n] = (u32)ci * chw16 + (u32)(slot % SPT) * 16u;
  }
  const u32 *posrow = postab + rg * (npos + 1) * 64 + lane;
  u32 yvoff[LY];  // the lane's offsets of the pixel loads about to be issued, read from the position table

  // per-channel addends of the blocks this wave writes back, fetched now so that the latency hides behind the loop
  int addv[S::NBW];
#pragma unroll
  for (int n = 0; n < S::NBW; ++n) {
    const int b = KG == 1 ? (wx * TX + n / TY) * S::YB : wave + n * S::NW;  // KG == 1: the wave's own blocks, NBW = TX * TY
    const int c = x0 + (b / S::YB) * 32 + l32;
    addv[n] = 0;
    if (c < ep.K) {
      if (ep.bias != nullptr) addv[n] = ep.bias[c];
      if constexpr (Q8) {
        if (ep.bias2 != nullptr) addv[n] += ep.bias2[c];
      }
    }
  }
  __syncthreads();  // position table visible

  int iss_off = 0;  // ring buffer (byte offset) of the stage whose loads are being issued
  auto bump = [](int off) { return off + S::STAGE == S::RING ? 0 : off + S::STAGE; };
  // offset of pixel load n (LX .. LW-1) out of the position table, to be read some MFMAs before the load is issued
  auto read_voff = [&](int n) {
    const int k = n - LX;
    const int row = ytap[k] < tap_end ? ypos[k] : npos;
    yvoff[k] = posrow[row * 64];
  };
  // direct load n (0 .. LW-1) of the stage being issued; advances the load's state to the next stage
  auto issue_one = [&](int n) {
    if (n < LX) {
      const int q = wg + n * S::NWG;
      if constexpr (F16) {
        dma_buffer_16(ring_addr + iss_off + q * 1024, xs[n] < s1 ? lane16 : kOutside, wsrc, (u32)(xsrc[n] - wgt));
      } else {
        const char *src = xs[n] < s1 ? xsrc[n] : zero;
        dma_global_16(ring_addr + iss_off + q * 1024, lane16, src);
      }
      xs[n] += KS;
      xsrc[n] += KS * 1024;
    } else {
      const int k = n - LX, q = wg + k * S::NWG;
      dma_buffer_16(ring_addr + iss_off + S::XPART + q * 1024, yvoff[k], rsrc, yci[k]);
      ytap[k] += TPS;
      ypos[k] += step_pos;
      yci[k] += (u32)step_ci * chw16;
      if (ypos[k] >= npos) {
        ypos[k] -= npos;
        yci[k] += chw16;
      }
    }
  };

  typename Op::acc_t acc[TX][TY];
#pragma unroll
  for (int i = 0; i < TX; ++i)
#pragma unroll
    for (int j = 0; j < TY; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  const int xfrag = (wx * TX) * 1024 + lane * 16;
  const int yfrag = S::XPART + (half * S::BY + (wy * TY) * 32 + l32) * 16;
  v4i xf[2][TX], yf[2][TY];
  // fragment idx of k-step ks of a stage: Y0, X0 (what the first MFMA needs), then the other Y, then the other X
  auto load_one = [&](const char *slot, int ks, int s, int idx) {
    const int j = idx == 0 ? 0 : idx - 1, i = idx == 1 ? 0 : idx - TY;
    if (idx == 0 || (idx >= 2 && idx <= TY))
      yf[s][j] = *reinterpret_cast<const v4i *>(slot + yfrag + (2 * ks * S::BY + j * 32) * 16);
    else
      xf[s][i] = *reinterpret_cast<const v4i *>(slot + xfrag + (ks * S::XB + i) * 1024);
  };
  // One k-step: every MFMA is followed by one slice of the stage's other work (a fragment read for the next
  // k-step, the table read or the issue of a direct load, the shift of the next pixel fragment) and a scheduling
  // fence.  s: fragment slot consumed; rd_slot / rd_ks: where the next k-step's fragments come from (has_read);
  // dl0: index of the first direct load this k-step issues, LPK of them (has_issue).
  auto step = [&](int s, const char *rd_slot, int rd_ks, int dl0, auto has_read, auto has_issue) {
    if constexpr (SHIFT) yf[s][0] ^= (int)0x80808080;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      const int i = m / TY, j = m % TY;
      acc[i][j] = Op::mma(xf[s][i], yf[s][j], acc[i][j]);
      if constexpr (decltype(has_read)::value) {
        if (m < NF) load_one(rd_slot, rd_ks, s ^ 1, m);
      }
      if constexpr (decltype(has_issue)::value) {
        if (m == 0) {
#pragma unroll
          for (int d = 0; d < LPK; ++d)
            if (dl0 + d >= LX && dl0 + d < LW) read_voff(dl0 + d);
        }
        if (m >= NM - LPK && dl0 + (m - (NM - LPK)) < LW) issue_one(dl0 + (m - (NM - LPK)));
      }
      if constexpr (SHIFT) {
        if (m + 1 < TY) yf[s][m + 1] ^= (int)0x80808080;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;

  // Stage st, computed from ring buffer cur_off.  AHEAD: stage st + NST - 1 exists and is fetched during this stage
  // (into iss_off); NEXT: stage st + 1 exists.
  int st = 0, cur_off = 0;
  auto stage = [&](auto ahead, auto next) {
    const char *cur = ring + cur_off;
    const int nxt_off = bump(cur_off);
    const char *nxt = ring + nxt_off;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS) {
        step(ks & 1, cur, ks + 1, ks * LPK, yes{}, ahead);
      } else {
        // stage st + 1 must have landed; the stages behind it and the loads of stage st + NST - 1 issued so far may
        // stay in flight.  Towards the end fewer stages are behind: `behind` counts the whole ones.
        constexpr int part = (KS - 1) * LPK < LW ? (KS - 1) * LPK : LW;
        if constexpr (decltype(ahead)::value) {
          UNIT_WAIT_VMCNT((NST - 3) * LW + part);
        } else {
          const int behind = nst - 2 - st;  // stages st + 2 .. nst - 1, all issued in full
          if (NST > 3 && behind >= NST - 3) {
            UNIT_WAIT_VMCNT((NST - 3) * LW);
          } else if (NST > 4 && behind == 2) {
            UNIT_WAIT_VMCNT(2 * LW);
          } else if (NST > 3 && behind == 1) {
            UNIT_WAIT_VMCNT(LW);
          } else {
            UNIT_WAIT_VMCNT(0);
          }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's reads of `cur` are done
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        step(ks & 1, nxt, 0, ks * LPK, next, ahead);
      }
    }
    if constexpr (decltype(ahead)::value) iss_off = bump(iss_off);
    cur_off = nxt_off;
    ++st;
  };

  // prologue: stages 0 .. NST - 2 by direct loads, the first fragments
#pragma unroll
  for (int p = 0; p < NST - 1; ++p)
    if (p < nst) {
#pragma unroll
      for (int n = LX; n < LW; ++n) read_voff(n);
#pragma unroll
      for (int n = 0; n < LW; ++n) issue_one(n);
      iss_off = bump(iss_off);
    }
  if (nst >= NST - 1) {
    UNIT_WAIT_VMCNT((NST - 2) * LW);
  } else {
    UNIT_WAIT_VMCNT(0);
  }
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < NF; ++i) load_one(ring, 0, 0, i);

  while (st + NST - 1 < nst) stage(yes{}, yes{});
  while (st + 1 < nst) stage(no{}, yes{});
  while (st < nst) stage(no{}, no{});
  // k-groups with fewer stages keep the others company at the barriers
  for (; st < rounds; ++st) __builtin_amdgcn_s_barrier();

  // ---- write-back (the rings are reused: everyone is past its last fragment read)
  __syncthreads();
  char *scratch = lds + S::kPark + wave * S::kScratch;
  int *wsb = reinterpret_cast<int *>(scratch + 32 * 144);
  const bool addend = ep.bias != nullptr || (Q8 && ep.bias2 != nullptr);
  if constexpr (KG == 1) {
#pragma unroll
    for (int i = 0; i < TX; ++i) {
      if (addend && half == 0) wsb[l32] = addv[i * TY];
#pragma unroll
      for (int j = 0; j < TY; ++j) {
        const int c0 = x0 + (wx * TX + i) * 32, m0 = y0 + (wy * TY + j) * 32;
        if constexpr (Q8)
          store_block_q8<Op>(ep, acc[i][j], addend ? wsb : nullptr, c0, m0, lane);
        else
          store_block<Op, NCHW>(ep, acc[i][j], addend ? wsb : nullptr, ep.scale, c0, m0, lane, scratch);
      }
    }
  } else {
    // every k-group parks its partial tile; then the blocks are dealt to all waves, which add the KG partial
    // blocks in k-group order (integer sums are exact in any order, fp32 sums the same from run to run) and write them
    using out4_t = typename Op::out4_t;
    char *mine = lds + grp * (S::BX * S::BY * 4);
#pragma unroll
    for (int i = 0; i < TX; ++i)
#pragma unroll
      for (int j = 0; j < TY; ++j) {
        const int b = (wx * TX + i) * S::YB + wy * TY + j;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<out4_t *>(mine + ((b * 4 + q) * 64 + lane) * 16) =
              out4_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
      }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < S::NBW; ++n) {
      const int b = wave + n * S::NW;
      if (b < S::NBLK) {
        typename Op::acc_t total;
#pragma unroll
        for (int r = 0; r < 16; ++r) total[r] = 0;
#pragma unroll
        for (int w = 0; w < KG; ++w) {
          const char *its = lds + w * (S::BX * S::BY * 4);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const out4_t v = *reinterpret_cast<const out4_t *>(its + ((b * 4 + q) * 64 + lane) * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) total[4 * q + e] += v[e];
          }
        }
        if (addend && half == 0) wsb[l32] = addv[n];
        const int c0 = x0 + (b / S::YB) * 32, m0 = y0 + (b % S::YB) * 32;
        if constexpr (Q8)
          store_block_q8<Op>(ep, total, addend ? wsb : nullptr, c0, m0, lane);
        else
          store_block<Op, NCHW>(ep, total, addend ? wsb : nullptr, ep.scale, c0, m0, lane, scratch);
      }
    }
  }
}

}  // namespace unit
