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
// consecutive rows each).  Zero padding is address selection: a lane whose tap falls outside the image
// fetches a 16-byte line of zeros instead (kept behind the prepared weights), so there are no masks on
// the data path; the u8 -> s8 shift is one XOR per fragment dword after the fragment read, its
// correction 128 * sum(w) comes precomputed with the prepared weights.
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

template <class S, bool SHIFT, bool Q8 = false, bool NCHW = false>
__global__ __launch_bounds__(S::NT) void conv_lds(const char *__restrict__ data, const char *__restrict__ wgt,
                                                  const char *__restrict__ zero, typename ConvEpilogue<OpI8>::Params ep,
                                                  ConvGeom g, GridMap gm, int nsteps) {
  using Op = OpI8;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int TX = S::TX, TY = S::TY, KG = S::KG, KS = S::KS, NST = S::NST, LW = S::LW, NM = S::NM, NF = S::NF;
  constexpr int LPK = S::LPK, LY = S::LY;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int grp = wave / S::NWG, wg = wave % S::NWG;
  const int wx = wg % S::WX, wy = wg / S::WX;
  const int l32 = lane & 31, half = lane >> 5;

  // k-steps [s0, s1) of this k-group, in stages of KS; every group runs `rounds` stages (one barrier each),
  // a group with fewer k-steps computes nothing in the surplus ones
  const int s0 = nsteps * grp / KG, s1 = nsteps * (grp + 1) / KG;
  const int rounds = ((nsteps + KG - 1) / KG + KS - 1) / KS;
  const int nst = (s1 - s0 + KS - 1) / KS;

  // tap (ci, kh, kw) -> (byte offset of the tap relative to the window origin, window position kh * KW + kw);
  // entries past the last tap point at position 31, which no pixel has inside: they fetch zeros
  v2i *tab = reinterpret_cast<v2i *>(lds + S::kMain);
  const int ntab = 2 * (nsteps + KG * KS);
  for (int e = threadIdx.x; e < ntab; e += S::NT) {
    v2i ent = {0, 31};
    if (e < g.ntaps) {
      int kw, rest, kh, ci;
      g.by_kw.divmod(e, rest, kw);
      g.by_kh.divmod(rest, ci, kh);
      ent[0] = ((ci * g.H + kh * g.dh) * g.W + kw * g.dw) * 16;
      ent[1] = kh * g.KW + kw;
    }
    tab[e] = ent;
  }

  int bx, by, split;
  gm.locate(blockIdx.x, bx, by, split);
  const int x0 = bx * S::BX, y0 = by * S::BY;
  char *ring = lds + grp * S::RING;

  // pixel side: this wave gathers rows rg * 64 + lane of the tile
  const int rg = wg % S::RG;
  u32 inside = 0;  // window positions (kh, kw) inside the image; none for rows past the last pixel
  int pixoff = 0;  // byte offset of the window origin (may lie before the tensor at the borders)
  {
    const int m = y0 + rg * 64 + lane;
    if (m < g.npix) {
      int n, rem, oh, ow;
      g.by_ohw.divmod(m, n, rem);
      g.by_ow.divmod(rem, oh, ow);
      const int ih0 = oh * g.sh - g.pt, iw0 = ow * g.sw - g.pl;
      pixoff = (int)(n * g.img_bytes) + (ih0 * g.W + iw0) * 16;
      u32 cols = 0, bits = 0;
      for (int kw = 0; kw < g.KW; ++kw) cols |= (u32)((u32)(iw0 + kw * g.dw) < (u32)g.W) << kw;
      for (int kh = 0; kh < g.KH; ++kh)
        if ((u32)(ih0 + kh * g.dh) < (u32)g.H) bits |= cols << (kh * g.KW);
      inside = bits;
    }
  }
  const int lastkb = (ep.K - 1) >> 5;
  const u32 lane16 = (u32)lane * 16u;
  // one of 256 lines of zeros, by workgroup and wave, so that the padded taps of the whole grid do not all queue
  // at one L2 channel
  const char *zline = zero + (((u32)blockIdx.x * 5u + (u32)wave * 3u) & 255u) * 64u;

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
  __syncthreads();  // tap table visible

  // the tap table entries of this wave's pixel loads for one stage, read ahead of their use
  v2i ent[LY];
  auto read_taps = [&](int st) {
    const int sb = s0 + st * KS;
#pragma unroll
    for (int n = 0; n < LY; ++n) ent[n] = tab[2 * sb + (wg + n * S::NWG) / S::RG];
  };
  // direct load n (0 .. LW-1) of this wave for stage st: first its share of the weight fragments, then of the
  // pixel rows (tap table entries in `ent`)
  auto issue_one = [&](int st, int n) {
    const int sb = s0 + st * KS;
    char *slot = ring + (st % NST) * S::STAGE;
    if (n < S::LX) {
      const int q = wg + n * S::NWG, ks = q / S::XB, xb = q % S::XB;
      int kb = (x0 >> 5) + xb;
      kb = kb < lastkb ? kb : lastkb;
      int s = sb + ks;
      s = s < nsteps - 1 ? s : nsteps - 1;  // surplus k-steps of a last stage re-read the last one; they are not computed
      const char *src = wgt + ((size_t)kb * nsteps + s) * 1024;
      __builtin_amdgcn_global_load_lds((gptr_t)(src + lane16), (lptr_t)(slot + q * 1024), 16, 0, 0);
    } else {
      const int q = wg + (n - S::LX) * S::NWG;
      const v2i e = ent[n - S::LX];
      const char *src = data + (u32)(pixoff + e[0]);
      src = ((inside >> e[1]) & 1u) ? src : zline;
      __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(slot + S::XPART + q * 1024), 16, 0, 0);
    }
  };

  v16i acc[TX][TY];
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
  // k-step, a direct load for stage issue_st, the shift of the next pixel fragment) and a scheduling fence.
  //   s: fragment slot consumed; rd_slot / rd_ks: where the next k-step's fragments come from (has_read);
  //   dl0: index of the first direct load this k-step issues, LPK of them (has_issue); live: the k-step counts
  auto step = [&](int s, const char *rd_slot, int rd_ks, int issue_st, int dl0, auto has_read, auto has_issue,
                  auto live) {
    if constexpr (SHIFT) yf[s][0] ^= (int)0x80808080;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      const int i = m / TY, j = m % TY;
      if constexpr (decltype(live)::value) acc[i][j] = Op::mma(xf[s][i], yf[s][j], acc[i][j]);
      if constexpr (decltype(has_read)::value) {
        if (m < NF) load_one(rd_slot, rd_ks, s ^ 1, m);
      }
      if constexpr (decltype(has_issue)::value) {
        if (m >= NM - LPK && dl0 + (m - (NM - LPK)) < LW) issue_one(issue_st, dl0 + (m - (NM - LPK)));
      }
      if constexpr (SHIFT) {
        if (m + 1 < TY) yf[s][m + 1] ^= (int)0x80808080;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;

  // Stage st.  AHEAD: stage st + NST - 1 exists and is fetched during this stage; NEXT: stage st + 1 exists.
  // The k-steps of the group's last stage that lie past s1 are skipped (the branch is uniform).
  auto stage = [&](int st, auto ahead, auto next) {
    const char *cur = ring + (st % NST) * S::STAGE;
    const char *nxt = ring + ((st + 1) % NST) * S::STAGE;
    const int sb = s0 + st * KS;
    if constexpr (decltype(ahead)::value) read_taps(st + NST - 1);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bool on = sb + ks < s1;
      if (ks + 1 < KS) {
        if (on)
          step(ks & 1, cur, ks + 1, st + NST - 1, ks * LPK, yes{}, ahead, yes{});
        else
          step(ks & 1, cur, ks + 1, st + NST - 1, ks * LPK, yes{}, ahead, no{});
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
        if (on)
          step(ks & 1, nxt, 0, st + NST - 1, ks * LPK, next, ahead, yes{});
        else
          step(ks & 1, nxt, 0, st + NST - 1, ks * LPK, next, ahead, no{});
      }
    }
  };

  // prologue: stages 0 .. NST - 2 by direct loads, the first fragments
#pragma unroll
  for (int p = 0; p < NST - 1; ++p)
    if (p < nst) {
      read_taps(p);
#pragma unroll
      for (int n = 0; n < LW; ++n) issue_one(p, n);
    }
  if (nst >= NST - 1) {
    UNIT_WAIT_VMCNT((NST - 2) * LW);
  } else {
    UNIT_WAIT_VMCNT(0);
  }
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < NF; ++i) load_one(ring, 0, 0, i);

  int st = 0;
  for (; st + NST - 1 < nst; ++st) stage(st, yes{}, yes{});
  for (; st + 1 < nst; ++st) stage(st, no{}, yes{});
  for (; st < nst; ++st) stage(st, no{}, no{});
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
    // blocks (integer sums: exact in any order) and write them
    char *mine = lds + grp * (S::BX * S::BY * 4);
#pragma unroll
    for (int i = 0; i < TX; ++i)
#pragma unroll
      for (int j = 0; j < TY; ++j) {
        const int b = (wx * TX + i) * S::YB + wy * TY + j;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<v4i *>(mine + ((b * 4 + q) * 64 + lane) * 16) =
              v4i{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
      }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < S::NBW; ++n) {
      const int b = wave + n * S::NW;
      if (b < S::NBLK) {
        v16i total;
#pragma unroll
        for (int r = 0; r < 16; ++r) total[r] = 0;
#pragma unroll
        for (int w = 0; w < KG; ++w) {
          const char *its = lds + w * (S::BX * S::BY * 4);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const v4i v = *reinterpret_cast<const v4i *>(its + ((b * 4 + q) * 64 + lane) * 16);
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
