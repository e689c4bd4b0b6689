// int8 dense with the reference's pre-packed weight, c (M, N) = a (M, K) u8 . W^T with
// wp[n/128][k/4][n%128][k%4] = W[n][k]:  activations go through LDS, weights straight from
// global memory into MFMA fragments.
//
// An experiment kept as a selectable variant.  The staged kernel moves both operand tiles through
// LDS, whose pipe (64 bytes per clock, writes and reads together) carries 4096 clocks of traffic
// per 256 x 256 x 128-byte stage against 2048 clocks of MFMA per SIMD; this kernel was written to
// test whether that is what bounds it.  It is not: with 1.6 x less LDS traffic the time is the
// same.  The pre-pack is fragment-shaped -- for one k-group (4 reduction bytes) the 128 n of a
// block are 512 contiguous bytes, so lane n reads its 16 reduction bytes of a k-step with four
// coalesced dword loads 512 bytes apart -- and weights are not shared between the lanes of a
// wave.  Taking them off the LDS leaves 32 KiB written + 128 KiB read per stage (2560 clocks)
// and puts 64 KiB on the L1 path instead.
//
// Tile<256, 256, 128, 2, 4>: 8 waves, wave tile 128 (m) x 64 (n).  Per stage (4 k-steps): the a
// tile of the next stage is written to the other LDS buffer, the one after that is fetched; the
// weight fragments of a k-step are consumed from a 4-slot register ring and re-fetched for the
// next stage.  Every load is unconditional (indices clamped, a rows past the end of the
// reduction staged as zeros), so the pipeline has no branches and the compiler's load waits
// leave exactly the younger loads in flight.
#pragma once
#include "epilogues.hpp"
#include "loaders.hpp"

namespace unit {

template <class T>
__global__ __launch_bounds__(T::NT) void gemm_mixed_i8(typename RowMajorLoader<T::BX, T::BKB, T::NT, true>::Params xp,
                                                       const char *__restrict__ wp, int N, int kg_total,
                                                       typename GemmEpilogue<OpI8, false>::Params ep, int nk, GridMap gm) {
  using XL = RowMajorLoader<T::BX, T::BKB, T::NT, true>;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int KK = T::BKB / 32, TX = T::TX, TY = T::TY;
  static_assert(KK == 4, "the weight ring has one slot per k-step of a 128-byte stage");
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wx = wave % T::WX, wy = wave / T::WX;
  const int l32 = lane & 31, half = lane >> 5;

  int bx, by, split;
  gm.locate(blockIdx.x, bx, by, split);
  const int x0 = bx * T::BX, y0 = by * T::BY;

  XL xl;
  xl.init(xp, x0, t, nullptr);

  // weights: byte offset of k-group 0 of this lane's n, per 32-column block (columns past N
  // re-read the last one; their results are never stored)
  u32 woff[TY];
#pragma unroll
  for (int j = 0; j < TY; ++j) {
    int n = y0 + wy * (TY * 32) + j * 32 + l32;
    n = n < N ? n : N - 1;
    woff[j] = (u32)(n >> 7) * (u32)kg_total * 512u + (u32)(n & 127) * 4u;
  }
  // a k-step takes k-groups 8 ks + 4 half + e, e = 0..3; a half past the end of the reduction
  // re-reads the last four k-groups: the matching a bytes are zeros, staged as -128, and
  // -128 * w in the accumulator cancels against +128 * w in the weight-sum correction
  const u32 wlast = (u32)(kg_total - 4) * 512u;
  const u32 whalf = (u32)half * 2048u;

  typename OpI8::acc_t acc[TX][TY];
#pragma unroll
  for (int i = 0; i < TX; ++i)
#pragma unroll
    for (int j = 0; j < TY; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  int wsx[TX], wsy[TY];
#pragma unroll
  for (int i = 0; i < TX; ++i) wsx[i] = 0;
#pragma unroll
  for (int j = 0; j < TY; ++j) wsy[j] = 0;

  const int xrow = wx * (TX * 32) + l32;
  const int xsw = swz<T::BKB>(xrow);
  const int xbase = xrow * T::BKB;
  v4i xf[2][TX];
  v4i wf[KK][TY];

  auto load_x = [&](const char *stage, int kk, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TX; ++i)
      xf[slot][i] = *reinterpret_cast<const v4i *>(stage + xbase + i * 32 * T::BKB + (((2 * kk + half) ^ xsw) << 4));
  };
  auto fetch_w = [&](auto slot, int ks) __attribute__((always_inline)) {
    constexpr int U = decltype(slot)::value;
    u32 kp = (u32)ks * 4096u + whalf;
    kp = kp < wlast ? kp : wlast;
#pragma unroll
    for (int j = 0; j < TY; ++j) {
      const u32 o = woff[j] + kp;
#pragma unroll
      for (int e = 0; e < 4; ++e) wf[U][j][e] = *reinterpret_cast<const int *>(wp + o + e * 512);
    }
  };
  auto mma_step = [&](int xslot, auto wslot) __attribute__((always_inline)) {
    constexpr int U = decltype(wslot)::value;
#pragma unroll
    for (int j = 0; j < TY; ++j)
#pragma unroll
      for (int d = 0; d < 4; ++d) wsy[j] = __builtin_amdgcn_sdot4(wf[U][j][d], 0x01010101, wsy[j], false);
#pragma unroll
    for (int i = 0; i < TX; ++i)
#pragma unroll
      for (int j = 0; j < TY; ++j) acc[i][j] = OpI8::mma(xf[xslot][i], wf[U][j], acc[i][j]);
  };

  // prologue: a stage 0 staged, a stage 1 and the weights of stage 0 in flight
  xl.template fetch<0>(0);
  xl.template commit<0>(lds);
  xl.template fetch<0>(1);
  fetch_w(std::integral_constant<int, 0>{}, 0);
  fetch_w(std::integral_constant<int, 1>{}, 1);
  fetch_w(std::integral_constant<int, 2>{}, 2);
  fetch_w(std::integral_constant<int, 3>{}, 3);
  __syncthreads();
  load_x(lds, 0, 0);

  for (int kt = 0; kt < nk; ++kt) {
    char *cur = lds + (kt & 1) * T::XBYTES;
    char *nxt = lds + ((kt & 1) ^ 1) * T::XBYTES;
    xl.template commit<0>(nxt);     // stage kt + 1 (zeros past the end)
    xl.template fetch<0>(kt + 2);
    auto step = [&](auto kkc) __attribute__((always_inline)) {
      constexpr int kk = decltype(kkc)::value;
      if constexpr (kk + 1 < KK) {
        load_x(cur, kk + 1, (kk + 1) & 1);
        mma_step(kk & 1, kkc);
      } else {
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();  // everyone has read `cur` and written `nxt`
        load_x(nxt, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        mma_step(kk & 1, kkc);
      }
      __builtin_amdgcn_sched_barrier(0);
      fetch_w(kkc, (kt + 1) * KK + kk);  // same k-step of the next stage into the slot just used
      __builtin_amdgcn_sched_barrier(0);
    };
    step(std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 1>{});
    step(std::integral_constant<int, 2>{});
    step(std::integral_constant<int, 3>{});
  }

#pragma unroll
  for (int j = 0; j < TY; ++j) wsy[j] += __shfl_xor(wsy[j], 32);

  GemmEpilogue<OpI8, false>::template store<T>(ep, acc, wsx, wsy, x0 + wx * (TX * 32), y0 + wy * (TY * 32), lane, wave,
                                                lds, false);
}

}  // namespace unit
