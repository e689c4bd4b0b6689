// NCHW16c convolution with both MFMA operands read straight from global memory into registers:
// no operand staging in LDS, no barrier in the reduction loop.
//
// Why: staging costs an LDS write and (wave tile permitting) several LDS reads per operand byte,
// all through one 64-byte-per-clock pipe, and that pipe -- not the matrix cores -- bounds the
// staged kernel whenever the output tile is small.  The layouts the reference uses happen to be
// MFMA fragments already (a lane holds 16 reduction bytes of one row per k-step):
//   * int8 data (N, C/16, H, W, 16) u8 / s8: the 16 channels of one pixel and tap are 16
//     contiguous bytes; consecutive lanes hold consecutive pixels (coalesced).  One k-step (32
//     bytes per row) = two taps: lanes 0-31 hold tap 2s, lanes 32-63 tap 2s+1;
//   * int8 weights (K/16, C/16, KH, KW, 4, 16, 4) s8: for one tap, channel kb of a 16-channel
//     block owns the dwords at kb*4 + e*64, e = 0..3: four dword loads per lane;
//   * fp16 data (N, C/16, H, W, 16): a pixel and tap are 32 bytes = one k-step; lanes 0-31 take
//     channels 0-7, lanes 32-63 channels 8-15;
//   * fp16 weights (K/16, C/16, KH, KW, 16 in, 16 out): out-channel o of a tap owns the halves at
//     o*2 + i*32: eight 16-bit loads per lane, packed in pairs by the load instruction.
//
// A workgroup is KG waves that all compute the same (32 TX channels) x (32 TY pixels) tile, each
// over its own share of the k-steps with a D-deep register prefetch ring; the partial tiles are
// summed in LDS and the waves share the write-back.
//
// The u8 operand is shifted to s8 (x ^ 0x80) for the signed MFMA and the kernel adds back
// 128 * sum(w), accumulated on the side with v_dot4 (SHIFT).  Signed data needs neither; that is
// the reference's fused form  (conv(x_s8 + 128, w) - 128 * sum(w) + bias) * scale
// (apps/cpu/relay/result.log:3-26), which the epilogue's bias and scale complete.
//
// PREP: the weights come in the fragment order written by prepare_weight (conv_prepare.hip)
// instead of the reference's layout: prepared[K/32][k-step][lane][16 bytes], so a lane's fragment of
// a k-step is one 16-byte load (a wave reads 1 KiB of consecutive memory) instead of four dword
// or eight 16-bit loads, and for u8 data the 128 * sum(w) correction is a per-channel constant
// that prepare_weight left behind the fragments (passed here as the bias), so the reduction loop
// does not accumulate weight sums.  The fragment that pads an odd tap count is zero.
//
// C4 (int8): data in 4-channel blocks (N, C/4, [D,] H, W, 4), the layout of the 3-channel stems.
// A pixel is 4 bytes, so the KW taps of one window row are consecutive memory: a k-step is one row
// (ci, kd, kh), lanes 0-31 hold its taps kw = 0..3 and lanes 32-63 kw = 4..7 (KW <= 8, no dilation
// along W).  Each tap is its own dword load with its own mask (row inside the image, per k-step;
// column inside the image and kw < KW, constant per lane), so no load leaves the tensor.  Taps
// kw >= KW carry masked data; their weights are zeros in prepared form, and with the reference's
// layout (K/16, C/4, [KD,] KH, KW, 1, 16, 4) they re-read tap KW - 1, which is harmless for the same
// reason as the odd tap above: masked data times any weight cancels (u8) or is zero (s8).
#pragma once
#include "epilogues.hpp"
#include "loaders.hpp"
#include "trace.hpp"

namespace unit {

// PAD: the convolution has zero padding, so taps can fall outside the image and are masked per
// lane; without it every tap of every valid pixel lies inside and the masking code is left out.
// D_ = ring depth, + 16 when the kernel is to be built for four waves per SIMD.
template <int TX_, int TY_, int KG_, int D_, bool PAD_ = true>
struct DirectShape {
  static constexpr int TX = TX_, TY = TY_, KG = KG_, D = D_ % 16;
  static constexpr bool PAD = PAD_;
  static constexpr int BX = TX * 32, BY = TY * 32;
  static constexpr int NT = 64 * KG;
  // One wave per tile and a two-deep ring: asked for four waves per SIMD the register allocator fits the kernel
  // into 128 VGPRs without spilling (it settles at 140 = three waves otherwise).  Deeper rings, wider tiles and
  // the per-tap loads of the reference's weight layout or of 4-channel blocks spill; the kernel asks only with
  // PREP && !C4.  A variant of its own, because it is not always a gain: short reductions with small outputs
  // run 0.6-0.9 us faster, the output-bound 1 x 1 64 -> 256 @56 layer 2 us slower.
  static constexpr bool kFourWaves = D_ >= 16;  // the variant asks for it (shown as "w4" in the variant name)
  static constexpr int kMinWavesPerSimd =
      (D_ >= 16 && KG == 1 && TX == 2 && TY == 2 && (D == 2 || (D == 3 && !PAD))) ? 4 : 1;  // three-deep: 127 VGPRs unpadded
  static constexpr int kScratch = 32 * 144 + 128;  // per wave: transpose area (32 pixels x 144-byte pitch) + 32 addends
  static constexpr int TILE = TX * TY * 4096;     // one 4-byte accumulator tile
  static constexpr int WSUM = TX * 32 * 4;        // summed 128 * weight sums
  // Integer partial tiles are added into one LDS tile with atomics (exact in any order).  Float
  // ones are parked side by side and the owner of a block adds them in wave order, so that results
  // do not vary from run to run.  (Parking integer tiles too was measured: fewer LDS instructions,
  // but KG tiles of LDS per workgroup leave room for one workgroup per CU, and layers with 1.5
  // tiles per CU lost 25 %.)
  template <class Op>
  static constexpr bool parked() {
    return !Op::kInt;
  }
  template <class Op>
  static constexpr int lds_fixed() {  // the tap table follows
    return KG * kScratch + (KG > 1 ? (parked<Op>() ? KG * (TILE + WSUM) : TILE + WSUM) : WSUM);
  }
  static_assert(NT <= 1024 && D >= 2 && D <= 8, "direct conv shape");
};

// Write one 32-channel x 32-pixel accumulator block to the (N, K/16, OH, OW, 16) output:
// transposed through the wave's LDS scratch so that 64 lanes store 16 pixels x 64 bytes = 1 KiB of
// consecutive output per instruction.  `wsb` (LDS, 32 values, or null) holds what is added per
// channel before the scale: the 128 * sum(w) correction and / or the bias.
// NCHW: planar (N, p.planar, OH, OW) output instead.  A template parameter and not a run-time branch:
// the branch, unrolled into the four blocks of a one-wave tile, cost every layer 16 VGPRs and 4 % of its time.
template <class Op, bool NCHW = false>
__device__ __forceinline__ void store_block(const typename ConvEpilogue<Op>::Params &p, const typename Op::acc_t &acc,
                                            const int *wsb, int scale, int c0, int m0, int lane, char *scratch) {
  using out4_t = typename Op::out4_t;
  using out_t = typename Op::out_t;
  constexpr int kPitch = 144;
  const int l32 = lane & 31, half = lane >> 5;
  const int rp = lane >> 2, piece = lane & 3;
  if constexpr (NCHW) {
    // (N, planar, OH, OW): register r of a lane is channel 8 (r / 4) + 4 half + r % 4 of the lane's pixel, so
    // a register of 32 lanes is 128 consecutive bytes of one channel plane: no transpose
    const int m = m0 + l32;
    int n, pix;
    p.by_ohw.divmod(m, n, pix);
    const __amdgpu_buffer_rsrc_t obuf = result_buffer(p.out);
    const u32 dst = (u32)(n * p.planar + c0 + 4 * half) * (u32)p.ohw + (u32)pix;  // in elements
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      out4_t v = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
      if constexpr (Op::kInt) {
        if (wsb) v += *reinterpret_cast<const v4i *>(wsb + 8 * q + 4 * half);
        if (scale != 1) v *= scale;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c0 + 8 * q + 4 * half + e < p.planar && m < p.npix)
          store_result(obuf, (dst + (u32)(8 * q + e) * (u32)p.ohw) * (u32)sizeof(out_t), v[e]);
    }
    return;
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    out4_t v = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
    if constexpr (Op::kInt) {
      if (wsb) v += *reinterpret_cast<const v4i *>(wsb + 8 * q + 4 * half);
      if (scale != 1) v *= scale;  // uniform; 32-bit integer multiplies run at a quarter of the VALU rate
    }
    *reinterpret_cast<out4_t *>(scratch + l32 * kPitch + (8 * q + 4 * half) * 4) = v;
  }
  const int ko_planes = p.K >> 4;
  const __amdgpu_buffer_rsrc_t obuf = result_buffer(p.out);
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int m = m0 + it * 16 + rp;
    int n, pix;
    p.by_ohw.divmod(m, n, pix);
    const u32 obase = ((u32)(n * ko_planes) * (u32)p.ohw + (u32)pix) * 16u + (u32)piece * 4u;  // in elements
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int c = c0 + h * 16;
      const out4_t v = *reinterpret_cast<const out4_t *>(scratch + (it * 16 + rp) * kPitch + h * 64 + piece * 16);
      if (c < p.K && m < p.npix)
        store_result(obuf, (obase + (u32)(c >> 4) * (u32)p.ohw * 16u) * (u32)sizeof(out_t), v);
    }
  }
}

// Requantised output: one 32-channel x 32-pixel int32 block -> u8 (N, K/16, OH, OW, 16),
//   q = clamp(((acc + addend[c]) * scale + 2^(shift-1)) >> shift, 0, 255)
// with the product and the shift in 64 bits.  A lane holds 16 channels of one pixel (4 h + 8 q + e);
// after packing each quad into a dword the two 32-lane halves swap two dwords each, so that half h
// holds the 16 bytes of plane c0 / 16 + h of its pixel: one 16-byte store per lane, 512 consecutive
// bytes per plane, no LDS.
template <class Op>
__device__ __forceinline__ void store_block_q8(const typename ConvEpilogue<Op>::Params &p, const v16i &acc, const int *wsb,
                                               int c0, int m0, int lane) {
  const int l32 = lane & 31, half = lane >> 5;
  int d[4];
  if (p.shift >= 33) {
    // The rounding term 2^(shift-1) is a multiple of 2^32, so it and the shift act on the high
    // dword of the product alone: floor((hi * 2^32 + lo + R) / 2^shift) = (hi + R / 2^32) >> (shift - 32).
    // (The host doubles scale and increments shift while that keeps scale in int32 -- the same
    // rational number -- so practical shifts arrive here.)
    const int rhi = 1 << (p.shift - 33), sh = p.shift - 32;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int t[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int v = acc[4 * q + e];
        if (wsb) v += wsb[8 * q + 4 * half + e];
        t[e] = __mulhi(v, p.scale) + rhi;
      }
      // v_ashr_pk_u8_i32: shift, saturate to 0..255 and pack two values into the low 16 bits (the
      // builtin's result is 16 bits wide; the upper half of the register is not zero, and the
      // byte select below never looks at it)
      const u32 lo = (unsigned short)__builtin_amdgcn_ashr_pk_u8_i32(t[0], t[1], sh);
      const u32 hi = (unsigned short)__builtin_amdgcn_ashr_pk_u8_i32(t[2], t[3], sh);
      d[q] = (int)__builtin_amdgcn_perm(hi, lo, 0x05040100u);
    }
  } else {
    const long long rnd = 1ll << (p.shift - 1);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      u32 packed = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int v = acc[4 * q + e];
        if (wsb) v += wsb[8 * q + 4 * half + e];
        long long t = ((long long)v * p.scale + rnd) >> p.shift;
        t = t < 0 ? 0 : (t > 255 ? 255 : t);
        packed |= (u32)t << (8 * e);
      }
      d[q] = (int)packed;
    }
  }
  // half 0 keeps d0, d1 (channels 0-3, 8-11) and needs the partner's d0, d1 (4-7, 12-15);
  // half 1 keeps d2, d3 (20-23, 28-31) and needs the partner's d2, d3 (16-19, 24-27)
  const int s0 = half ? d[0] : d[2], s1 = half ? d[1] : d[3];
  const int r0 = __shfl_xor(s0, 32), r1 = __shfl_xor(s1, 32);
  const v4i row = half ? v4i{r0, d[2], r1, d[3]} : v4i{d[0], r0, d[1], r1};
  const int m = m0 + l32, c = c0 + half * 16;
  if (c < p.K && m < p.npix) {
    int n, pix;
    p.by_ohw.divmod(m, n, pix);
    store_result(result_buffer(p.out), (((u32)(n * (p.K >> 4)) + (u32)(c >> 4)) * (u32)p.ohw + (u32)pix) * 16u, row);
  }
}

template <class Op, class S, bool SHIFT, bool PREP = false, bool C4 = false, bool Q8 = false, bool NCHW = false>
__global__ __launch_bounds__(S::NT) __attribute__((amdgpu_waves_per_eu(PREP && !C4 ? S::kMinWavesPerSimd : 1))) void conv_direct(const char *__restrict__ data, const char *__restrict__ wgt,
                                                     typename ConvEpilogue<Op>::Params ep, ConvGeom g, GridMap gm
                                                     UNIT_TRACE(, unsigned long long *trace_buf)) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int TX = S::TX, TY = S::TY, KG = S::KG, D = S::D;
  // timeline: 0 entry, 1 arguments fetched, 2 the ring's weight loads issued, 3 per-lane window state built, 4 the
  // ring's pixel loads issued, 5 reduction done (accumulators complete), 6 k-groups summed, 7 stores issued and
  // acknowledged
  UNIT_TRACE(WaveTrace tr; tr.mark(0);)
  {
    // Touch each of the five 64-byte lines of kernel arguments at once: the compiler fetches the arguments
    // where it first needs them, in three dependent rounds of scalar loads before the first operand fetch.
    const auto *ka = (const __attribute__((address_space(4))) int *)__builtin_amdgcn_kernarg_segment_ptr();
    const int w0 = ka[0], w1 = ka[16], w2 = ka[32], w3 = ka[48], w4 = ka[64];
    asm volatile("" ::"s"(w0), "s"(w1), "s"(w2), "s"(w3), "s"(w4));
  }
  UNIT_TRACE(tr.mark(1);)
  constexpr bool kInt = Op::kInt;
  constexpr int TAPB = C4 ? 4 : (kInt ? 16 : 32);  // bytes of one pixel and tap
  constexpr int WTAP = kInt ? 256 : 512;           // bytes of one tap of a 16-channel weight block
  static_assert(kInt || (!SHIFT && !S::PAD), "the fp16 operator has neither a shift nor padding");
  static_assert(!C4 || (kInt && S::PAD), "4-channel blocks: int8, masked loads");
  static_assert(!Q8 || kInt, "requantised output is an int8 operator");
  static_assert(!NCHW || (kInt && !Q8), "planar output: the int32 fused form");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int l32 = lane & 31, half = lane >> 5;

  char *scratch = lds + wave * S::kScratch;
  char *tiles = lds + KG * S::kScratch;
  constexpr bool kParked = KG > 1 && S::template parked<Op>();
  // the per-channel addends: one row, or one per wave when the tiles are parked
  int *wsum = reinterpret_cast<int *>(lds + S::template lds_fixed<Op>() - (kParked ? KG : 1) * S::WSUM);
  v2i *tab = reinterpret_cast<v2i *>(lds + S::template lds_fixed<Op>());

  // tap (ci, kd, kh, kw) -> (byte offset of the tap inside an image relative to the window origin,
  // index of its window position kh * KW + kw).  int8 pairs taps into k-steps: the odd tap past the end points
  // at bit 31 of the window set, which is never set, so it is staged like zero padding.
  // C4: a k-step is (channel block, kh); the table holds the row's offset for both halves and kh
  const int nsteps = C4 ? g.c4_steps : (kInt ? (g.ntaps + 1) >> 1 : g.ntaps);
  const int ntab = kInt ? 2 * nsteps : nsteps;
  auto tap_entry = [&](int e) __attribute__((always_inline)) {
    v2i ent = {0, 31};
    if constexpr (C4) {
      int rest, kh;
      g.by_kh.divmod(e >> 1, rest, kh);
      int ci = rest, kd = 0;
      if (g.KD > 1) g.by_kd.divmod(rest, ci, kd);
      ent[0] = (((ci * g.D + kd) * g.H + kh * g.dh) * g.W) * 4 + (e & 1) * 16;
      ent[1] = g.nopad ? 0 : kh;
    } else if (e < g.ntaps) {
      // (the dividers by one are skipped: each costs two quarter-rate multiplies on the way to the first loads)
      int kw = 0, rest = e, kh = 0;
      if (g.KW > 1) g.by_kw.divmod(e, rest, kw);
      int rest2 = rest;
      if (g.KH > 1) g.by_kh.divmod(rest, rest2, kh);
      int ci = rest2, kd = 0;
      if (g.KD > 1) g.by_kd.divmod(rest2, ci, kd);
      ent[0] = (((ci * g.D + kd) * g.H + kh * g.dh) * g.W + kw * g.dw) * TAPB;
      ent[1] = g.nopad ? 0 : kh * g.KW + kw;
    }
    return ent;
  };

  // The prologue is ordered by what the first loads need, because a wave's life at batch 32 is a chain of
  // latencies rather than a rate: the ring's weight fragments depend on the workgroup's place alone and go out
  // first; the ring's pixel fragments need this lane's window origin and the ring's own tap entries, which lane q
  // computes for tap q of the ring and the wave reads back lane by lane; the tap table in LDS, the zeroed sums and the
  // barrier that publishes them are only needed by the fetches after the ring and follow the loads.
  int bx, by, split;
  gm.locate(blockIdx.x, bx, by, split);
  const int x0 = bx * S::BX, y0 = by * S::BY;

  // weights: byte offset of this lane's share of its channel's tap 0, per 32-channel block (rows
  // past K re-read the last channel; their results are never stored)
  u32 xoff[TX];
#pragma unroll
  for (int i = 0; i < TX; ++i) {
    int n = x0 + i * 32 + l32;
    n = n < ep.K ? n : ep.K - 1;
    xoff[i] = (u32)(n >> 4) * (u32)(g.ntaps * WTAP) + (kInt ? (u32)(n & 15) * 4u : (u32)(n & 15) * 2u + (u32)half * 256u);
    if constexpr (PREP) {  // blocks past the last one re-read it
      const int kb = min((x0 >> 5) + i, (ep.K - 1) >> 5);
      xoff[i] = ((u32)(kb * nsteps) * 64u + (u32)lane) * 16u;
    } else if constexpr (C4) {  // a tap of a 16-channel block is 64 bytes, a window row KW of them
      xoff[i] = (u32)(n >> 4) * (u32)(g.ntaps * 64) + (u32)(n & 15) * 4u;
    }
  }
  // C4 on the reference's weight layout: byte offset of this lane's four taps inside a window row
  u32 wtap[C4 && !PREP ? 4 : 1];
  if constexpr (C4 && !PREP) {
#pragma unroll
    for (int e = 0; e < 4; ++e) wtap[e] = (u32)min(4 * half + e, g.KW - 1) * 64u;
  }
  auto for_slots = [&](auto f) __attribute__((always_inline)) {
    f(std::integral_constant<int, 0>{});
    f(std::integral_constant<int, 1>{});
    if constexpr (D > 2) f(std::integral_constant<int, 2>{});
    if constexpr (D > 3) f(std::integral_constant<int, 3>{});
    if constexpr (D > 4) f(std::integral_constant<int, 4>{});
    if constexpr (D > 5) f(std::integral_constant<int, 5>{});
    if constexpr (D > 6) f(std::integral_constant<int, 6>{});
    if constexpr (D > 7) f(std::integral_constant<int, 7>{});
  };

  // prefetch ring: D k-steps of fragments in registers
  v4i xf[D][TX], yf[D][TY];
  int ym[S::PAD && !C4 ? D : 1][TY];  // all ones where the tap lies inside the image, else 0
  v4i ym4[C4 ? D : 1][TY];           // C4: the same per tap of the fragment
  const u32 last_tap_off = (u32)(g.ntaps - 1) * (u32)WTAP;

  // this wave's k-steps [s0, s1); fetches past the last one re-read it
  const int s0 = nsteps * wave / KG, s1 = nsteps * (wave + 1) / KG;
  const int slast = s1 - 1;

  // Offsets are unsigned 32-bit values added to a uniform base pointer, so a load needs no 64-bit
  // address arithmetic per lane.
  // The weight fragments of k-step `scur`.
  auto fetch_w = [&](auto slot, int scur) __attribute__((always_inline)) {
    constexpr int U = decltype(slot)::value;
    const int t = kInt ? 2 * scur + half : scur;
    const u32 xs = (u32)scur * 1024u;  // PREP: a k-step of a 32-channel block is 1 KiB
    // int8: the odd tap past the end re-reads the last tap's weights.  Its data is staged as
    // zero padding, and a padded position contributes -128 * w to the accumulator and +128 * w
    // through the weight-sum correction (SHIFT) or 0 * w (signed data), whatever w is.
    u32 xk = (u32)t * (u32)WTAP;
    xk = xk < last_tap_off ? xk : last_tap_off;
#pragma unroll
    for (int i = 0; i < TX; ++i) {
      const u32 o = xoff[i] + xk;
      if constexpr (PREP) {
        xf[U][i] = *reinterpret_cast<const v4i *>(wgt + (xoff[i] + xs));
      } else if constexpr (C4) {
        const u32 xr = (u32)scur * (u32)(g.KW * 64);  // this k-step's window row
#pragma unroll
        for (int d = 0; d < 4; ++d) xf[U][i][d] = *reinterpret_cast<const int *>(wgt + (xoff[i] + xr + wtap[d]));
      } else if constexpr (kInt) {
#pragma unroll
        for (int d = 0; d < 4; ++d) xf[U][i][d] = *reinterpret_cast<const int *>(wgt + o + d * 64);
      } else {
        v8h h;
#pragma unroll
        for (int k = 0; k < 8; ++k) h[k] = *reinterpret_cast<const _Float16 *>(wgt + o + k * 32);
        xf[U][i] = __builtin_bit_cast(v4i, h);
      }
    }
  };
  if (s0 < s1) {
    for_slots([&](auto u) __attribute__((always_inline)) {
      fetch_w(u, min(s0 + decltype(u)::value, slast));
    });
  }
  __builtin_amdgcn_sched_barrier(0);
  UNIT_TRACE(tr.mark(2);)

  // data: byte offset of the window origin of this lane's pixel per 32-pixel block, and the set of
  // window positions (kh, kw) that fall inside the image (none for lanes past the last pixel)
  int pixoff[TY];
  u32 inside[TY];
  v4i colm[C4 ? TY : 1];  // C4: per tap of this lane's half, all ones if its column is inside the image and kw < KW
#pragma unroll
  for (int j = 0; j < TY; ++j) {
    const int m = y0 + j * 32 + l32;
    pixoff[j] = (kInt || C4) ? 0 : half * 16;
    inside[j] = 0;
    if constexpr (C4) colm[j] = v4i{0, 0, 0, 0};
    if (m < g.npix) {
      int n, rem, oh, ow;
      g.by_ohw.divmod(m, n, rem);
      int od = 0, rem2 = rem;  // a 2-D convolution
      if (g.D > 1) g.by_plane.divmod(rem, od, rem2);
      g.by_ow.divmod(rem2, oh, ow);
      const int ih0 = oh * g.sh - g.pt, iw0 = ow * g.sw - g.pl;
      pixoff[j] += (int)(n * g.img_bytes) + ((od * g.sd * g.H + ih0) * g.W + iw0) * TAPB;
      if constexpr (C4) {
        u32 rows = 0;  // rows kh inside the image
        for (int kh = 0; kh < g.KH; ++kh) rows |= (u32)((u32)(ih0 + kh * g.dh) < (u32)g.H) << kh;
        inside[j] = g.nopad ? 1u : rows;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int kw = 4 * half + e;
          colm[j][e] = (kw < g.KW && (u32)(iw0 + kw) < (u32)g.W) ? -1 : 0;
        }
      } else if constexpr (S::PAD) {
        u32 cols = 0, bits = 0;  // columns kw inside the image; then one copy of them per row kh inside
        if (g.row_ones) {  // undilated: columns [ka, kb) and rows [ra, rb) of the window are inside
          const int ka = min(max(-iw0, 0), g.KW), kb = min(max(g.W - iw0, ka), g.KW);
          const int ra = min(max(-ih0, 0), g.KH), rb = min(max(g.H - ih0, ra), g.KH);
          cols = (1u << kb) - (1u << ka);
          bits = cols * (g.row_ones & ((1u << (rb * g.KW)) - (1u << (ra * g.KW))));
        } else {
          for (int kw = 0; kw < g.KW; ++kw) cols |= (u32)((u32)(iw0 + kw * g.dw) < (u32)g.W) << kw;
          for (int kh = 0; kh < g.KH; ++kh)
            if ((u32)(ih0 + kh * g.dh) < (u32)g.H) bits |= cols << (kh * g.KW);
        }
        inside[j] = g.nopad ? 1u : bits;  // without padding every real tap carries position 0
      }
    }
  }
  UNIT_TRACE(asm volatile("s_nop 0" ::"v"(pixoff[0]), "v"(inside[0])); tr.mark(3);)

  // The pixel fragments of one k-step, whose tap table entry for this lane's half is `e`.
  auto fetch_d = [&](auto slot, v2i e) __attribute__((always_inline)) {
    constexpr int U = decltype(slot)::value;
#pragma unroll
    for (int j = 0; j < TY; ++j) {
      if constexpr (C4) {
        const int rowm = __builtin_amdgcn_sbfe((int)inside[j], (u32)e[1], 1u);
        const u32 o = (u32)(pixoff[j] + e[0]);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int m = rowm & colm[j][d];
          // the sum is formed in 32 bits before masking: o alone may lie before the tensor (left edge of row 0)
          yf[U][j][d] = *reinterpret_cast<const int *>(data + ((o + (u32)(d * 4)) & (u32)m));
          ym4[U][j][d] = m;
        }
      } else if constexpr (S::PAD) {
        // all ones if window position e[1] of this lane's pixel is inside the image, else 0
        const int m = __builtin_amdgcn_sbfe((int)inside[j], (u32)e[1], 1u);
        yf[U][j] = *reinterpret_cast<const v4i *>(data + ((u32)(pixoff[j] + e[0]) & (u32)m));
        ym[U][j] = m;
      } else {
        yf[U][j] = *reinterpret_cast<const v4i *>(data + (u32)(pixoff[j] + e[0]));
      }
    }
  };
  if (s0 < s1) {
    // lane q holds the entry of the ring's tap q (int8: two taps per k-step, one per half of the wave)
    const int e0 = kInt ? 2 * s0 : s0;
    const v2i mine = e0 + lane < ntab ? tap_entry(e0 + lane) : v2i{0, 31};
    for_slots([&](auto u) __attribute__((always_inline)) {
      const int q = min((int)decltype(u)::value, slast - s0);  // uniform
      v2i e;
      if constexpr (kInt) {
        const int a0 = __builtin_amdgcn_readlane(mine[0], 2 * q), a1 = __builtin_amdgcn_readlane(mine[1], 2 * q);
        const int b0 = __builtin_amdgcn_readlane(mine[0], 2 * q + 1), b1 = __builtin_amdgcn_readlane(mine[1], 2 * q + 1);
        e = half ? v2i{b0, b1} : v2i{a0, a1};
      } else {
        e = v2i{__builtin_amdgcn_readlane(mine[0], q), __builtin_amdgcn_readlane(mine[1], q)};
      }
      fetch_d(u, e);
    });
  }
  __builtin_amdgcn_sched_barrier(0);
  UNIT_TRACE(tr.mark(4);)

  // per-channel addend read from memory (bias; with PREP and u8 data the shift correction): one
  // wave contributes it, and the load is issued here so that its latency hides behind the loop
  int addv[TX];
#pragma unroll
  for (int i = 0; i < TX; ++i) {
    addv[i] = 0;
    if constexpr (kInt) {
      const int c = x0 + i * 32 + l32;
      if (ep.bias != nullptr && wave == 0 && c < ep.K) addv[i] = ep.bias[c];
      if constexpr (Q8) {
        if (ep.bias2 != nullptr && wave == 0 && c < ep.K) addv[i] += ep.bias2[c];
      }
    }
  }
  // the tap table for the fetches after the ring -- not built, and its barrier not taken, when no wave of the
  // workgroup has more k-steps than the ring holds -- and the zeroed sums
  const bool need_tab = (nsteps + KG - 1) / KG > D;
  if (need_tab)
    for (int e = threadIdx.x; e < ntab; e += S::NT) tab[e] = tap_entry(e);
  if constexpr (KG > 1 && !kParked) {
    v4i *z = reinterpret_cast<v4i *>(tiles);
    for (int e = threadIdx.x; e < (S::TILE + S::WSUM) / 16; e += S::NT) z[e] = v4i{0, 0, 0, 0};
  }

  typename Op::acc_t acc[TX][TY];
#pragma unroll
  for (int i = 0; i < TX; ++i)
#pragma unroll
    for (int j = 0; j < TY; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  int wsx[TX];
#pragma unroll
  for (int i = 0; i < TX; ++i) wsx[i] = 0;

  // Fetches after the ring run through the k-steps in order; `sf` is the next one (it stops at the wave's last
  // k-step, so surplus fetches re-read that one) and `ecur` its tap table entry, read one fetch
  // ahead so that the LDS latency is not in the way of the loads.
  int sf = 0;
  v2i ecur = {0, 31};
  auto fetch = [&](auto slot) __attribute__((always_inline)) {
    const int scur = sf;
    const v2i e = ecur;
    sf = sf < slast ? sf + 1 : slast;
    ecur = tab[kInt ? 2 * sf + half : sf];
    fetch_w(slot, scur);
    fetch_d(slot, e);
  };
  auto consume = [&](auto slot) __attribute__((always_inline)) {
    constexpr int U = decltype(slot)::value;
    v4i y[TY];
#pragma unroll
    for (int j = 0; j < TY; ++j)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        int v = yf[U][j][d];
        if constexpr (C4)
          v &= ym4[U][j][d];
        else if constexpr (S::PAD)
          v &= ym[U][j];
        if constexpr (SHIFT) v ^= (int)0x80808080;
        y[j][d] = v;
      }
    if constexpr (SHIFT && !PREP) {
#pragma unroll
      for (int i = 0; i < TX; ++i)
#pragma unroll
        for (int d = 0; d < 4; ++d) wsx[i] = __builtin_amdgcn_sdot4(xf[U][i][d], 0x01010101, wsx[i], false);
    }
#pragma unroll
    for (int i = 0; i < TX; ++i)
#pragma unroll
      for (int j = 0; j < TY; ++j) acc[i][j] = Op::mma(xf[U][i], y[j], acc[i][j]);
  };

  if (need_tab) __syncthreads();  // tap table (and the zeroed sums) visible

  // Software pipeline over this wave's k-steps.  Every path issues the same loads in the
  // same (slot) order and only the consumes are conditional, so the wait the compiler places
  // before a consume always leaves the D - 1 younger slots in flight.  (With conditional
  // fetches the wait has to cover the path on which the slot is the youngest load and becomes
  // "wait for everything".)  The price: fetches past the end re-read the last k-step.
  // The sched_barriers keep consume(u) -> fetch(u) in program order; left alone, the scheduler
  // gathers the loads of all D slots at the end of the loop body.
  // The first round stands outside the loop: the ring was issued weights first, then pixels, and a loop head that
  // merges that order with the loop's own would make every round wait as if the ring's order still held.
  if (s0 < s1) {
    sf = min(s0 + D, slast);
    if (need_tab) ecur = tab[kInt ? 2 * sf + half : sf];
    auto round = [&]() __attribute__((always_inline)) {
      for_slots([&](auto u) __attribute__((always_inline)) {
        consume(u);
        __builtin_amdgcn_sched_barrier(0);
        fetch(u);
        __builtin_amdgcn_sched_barrier(0);
      });
    };
    int s = s0;
    // while more than D k-steps remain: consume a round and fetch the next one (in the last round fewer than D
    // k-steps are new; the surplus fetches repeat the wave's last k-step)
    if (s + D < s1) {
      round();
      for (s += D; s + D < s1; s += D) round();
    }
    for_slots([&](auto u) __attribute__((always_inline)) {  // 1 .. D k-steps left, all in flight
      if (s + decltype(u)::value < s1) consume(u);
      __builtin_amdgcn_sched_barrier(0);
    });
  }

  UNIT_TRACE(asm volatile("s_nop 0" ::"v"(acc[TX - 1][TY - 1][15])); tr.mark(5);)
  // the two 32-lane halves hold the weight sums of the two taps of every k-step
  if constexpr (SHIFT && !PREP) {
#pragma unroll
    for (int i = 0; i < TX; ++i) wsx[i] = (wsx[i] + __shfl_xor(wsx[i], 32)) << 7;
  }
  // what is added per channel before the scale: the shift correction and / or the bias; one wave
  // adds the bias.  `addend` is uniform over the workgroup.
  const bool addend = kInt && (SHIFT || ep.bias != nullptr || (Q8 && ep.bias2 != nullptr));
#pragma unroll
  for (int i = 0; i < TX; ++i) wsx[i] += addv[i];

  if constexpr (KG == 1) {
    if (addend && half == 0) {
#pragma unroll
      for (int i = 0; i < TX; ++i) wsum[i * 32 + l32] = wsx[i];
    }
#pragma unroll
    for (int i = 0; i < TX; ++i)
#pragma unroll
      for (int j = 0; j < TY; ++j)
        if constexpr (Q8)
          store_block_q8<Op>(ep, acc[i][j], addend ? wsum + i * 32 : nullptr, x0 + i * 32, y0 + j * 32, lane);
        else
          store_block<Op, NCHW>(ep, acc[i][j], addend ? wsum + i * 32 : nullptr, ep.scale, x0 + i * 32, y0 + j * 32, lane,
                          scratch);
  } else if constexpr (!kParked) {
    // sum the partial tiles of the KG waves in LDS, then share the blocks among the waves
    if (!need_tab) __syncthreads();  // the zeroed sums, when the barrier before the reduction was not taken
    int *sum = reinterpret_cast<int *>(tiles);
#pragma unroll
    for (int i = 0; i < TX; ++i)
#pragma unroll
      for (int j = 0; j < TY; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          __hip_atomic_fetch_add(sum + ((i * TY + j) * 16 + r) * 64 + lane, acc[i][j][r], __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_WORKGROUP);
    if (addend && half == 0) {
#pragma unroll
      for (int i = 0; i < TX; ++i)
        __hip_atomic_fetch_add(wsum + i * 32 + l32, wsx[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
    UNIT_TRACE(tr.mark(6);)
    for (int b = wave; b < TX * TY; b += KG) {
      const int i = b / TY, j = b - i * TY;
      v16i total;
#pragma unroll
      for (int r = 0; r < 16; ++r) total[r] = sum[(b * 16 + r) * 64 + lane];
      if constexpr (Q8)
        store_block_q8<Op>(ep, total, addend ? wsum + i * 32 : nullptr, x0 + i * 32, y0 + j * 32, lane);
      else
        store_block<Op, NCHW>(ep, total, addend ? wsum + i * 32 : nullptr, ep.scale, x0 + i * 32, y0 + j * 32, lane, scratch);
    }
  } else {
    // every wave parks its partial tile (and addends); the owner of a block adds them in wave order
    using out4_t = typename Op::out4_t;
    char *mine = tiles + wave * S::TILE;
#pragma unroll
    for (int i = 0; i < TX; ++i)
#pragma unroll
      for (int j = 0; j < TY; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<out4_t *>(mine + (((i * TY + j) * 4 + q) * 64 + lane) * 16) =
              out4_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
    if constexpr (kInt) {
      if (addend && half == 0) {
#pragma unroll
        for (int i = 0; i < TX; ++i) wsum[wave * (TX * 32) + i * 32 + l32] = wsx[i];
      }
    }
    __syncthreads();
    for (int b = wave; b < TX * TY; b += KG) {
      const int i = b / TY, j = b - i * TY;
      typename Op::acc_t total;
#pragma unroll
      for (int r = 0; r < 16; ++r) total[r] = 0;
      for (int w = 0; w < KG; ++w) {
        const char *its = tiles + w * S::TILE;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const out4_t v = *reinterpret_cast<const out4_t *>(its + ((b * 4 + q) * 64 + lane) * 16);
#pragma unroll
          for (int e = 0; e < 4; ++e) total[4 * q + e] += v[e];
        }
      }
      if constexpr (kInt) {
        // the block's addends of all waves, summed into row 0 by the lanes that hold them
        if (addend && half == 0) {
          int a = 0;
          for (int w = 0; w < KG; ++w) a += wsum[w * (TX * 32) + i * 32 + l32];
          reinterpret_cast<int *>(scratch)[1152 + l32] = a;  // behind the transpose area
        }
        store_block<Op, NCHW>(ep, total, addend ? reinterpret_cast<const int *>(scratch) + 1152 : nullptr, ep.scale,
                        x0 + i * 32, y0 + j * 32, lane, scratch);
      } else {
        store_block<Op, NCHW>(ep, total, nullptr, 1, x0 + i * 32, y0 + j * 32, lane, scratch);
      }
    }
  }
  UNIT_TRACE(__builtin_amdgcn_s_waitcnt(0x0F70); tr.mark(7); tr.flush(trace_buf, blockIdx.x * KG + wave);)
}

}  // namespace unit
