// Accumulator write-back for mma_kernel.  Outputs are written once and never read back by the
// kernel, so they go out as agent-scope non-temporal stores (store_result, mma_core.hpp): the lines
// neither stay dirty in the L2 until the write-back at the end of the kernel nor displace the next
// launches' operands in the memory-side cache.
#pragma once
#include "mma_core.hpp"

namespace unit {

// Row-major C (M, N): X rows are m, Y rows are n.  A lane holds one n (l % 32) and 16 m values,
// so each store instruction writes two 128-byte row segments.  For int8 the weight is the Y
// operand: out = acc + 128 * sum_k w[n][k].
template <class Op, bool OUT_F16>
struct GemmEpilogue {
  static constexpr bool kSplitPlanes = false;
  struct Params {
    void *c;
    int M, N;
  };
  template <class T>
  static constexpr int lds_bytes() {
    return 0;
  }
  template <class T>
  static __device__ __forceinline__ void store(const Params &p, typename Op::acc_t (&acc)[T::TX][T::TY],
                                               int (&)[T::TX], int (&wsy)[T::TY], int xw0, int yw0, int lane,
                                               int, char *, bool accumulate, int yrot = 0) {
    // yrot: accumulator column j (and wsy[j]) belongs to Y block (j + yrot) % TY of the wave tile
    const int l32 = lane & 31, half = lane >> 5;
    const __amdgpu_buffer_rsrc_t cbuf = result_buffer(p.c);
#pragma unroll
    for (int j = 0; j < T::TY; ++j) {
      const int n = yw0 + ((j + yrot) % T::TY) * 32 + l32;
      if (n >= p.N) continue;
#pragma unroll
      for (int i = 0; i < T::TX; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = xw0 + i * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
          if (m >= p.M) continue;
          const size_t idx = (size_t)m * p.N + n;
          if constexpr (Op::kInt) {
            const int v = acc[i][j][r] + (wsy[j] << 7);
            if (accumulate)
              atomicAdd(reinterpret_cast<int *>(p.c) + idx, v);
            else
              store_result(cbuf, (u32)idx * 4u, v);
          } else if constexpr (OUT_F16) {
            store_result(cbuf, (u32)idx * 2u, (_Float16)acc[i][j][r]);  // no k-splits for f16 out
          } else {
            if (accumulate)
              unsafeAtomicAdd(reinterpret_cast<float *>(p.c) + idx, acc[i][j][r]);
            else
              store_result(cbuf, (u32)idx * 4u, acc[i][j][r]);
          }
        }
    }
  }
};

// k-splits without atomics: split s of the fp16 GEMM writes its partial tile as plain fp32 stores into plane s of a
// workspace (M * N floats each); a second kernel adds the planes in split order, so the result does not depend on
// which workgroup finishes first, and can be rounded to fp16 afterwards.
struct GemmPlaneEpilogue {
  static constexpr bool kSplitPlanes = true;
  struct Params {
    void *c;  // plane 0 of the workspace
    int M, N;
    size_t plane;  // bytes per plane
  };
  template <class T>
  static constexpr int lds_bytes() {
    return 0;
  }
  template <class T>
  static __device__ __forceinline__ void store(const Params &p, typename OpF16::acc_t (&acc)[T::TX][T::TY], int (&wsx)[T::TX],
                                               int (&wsy)[T::TY], int xw0, int yw0, int lane, int wave, char *lds, int split) {
    typename GemmEpilogue<OpF16, false>::Params q{static_cast<char *>(p.c) + (size_t)split * p.plane, p.M, p.N};
    GemmEpilogue<OpF16, false>::template store<T>(q, acc, wsx, wsy, xw0, yw0, lane, wave, lds, false);
  }
};

// Convolution output (N, K/16, OH, OW, 16), 4-byte elements: X rows are output channels, Y rows
// are output pixels.  In the accumulators a lane holds one pixel and, per register quad, 4
// consecutive channels; written like that, a store instruction would scatter 16-byte pieces over
// 32 pixels.  Each wave therefore transposes one 32 x 32 block at a time through its own LDS
// scratch (32 pixels x 144-byte pitch, conflict-free 16-byte writes) and reads it back so that 64
// lanes cover 16 pixels x 64 bytes = 1 KiB of consecutive output per store instruction.
// LDS operations of one wave execute in order, so the scratch needs no barrier.
// For int8 the weight is the X operand; its per-channel sums live in other lanes and go through
// the same per-wave LDS area once.
template <class Op>
struct ConvEpilogue {
  static constexpr bool kSplitPlanes = false;
  struct Params {
    void *out;
    int K;     // output channels (multiple of 16)
    int ohw;   // OH * OW
    int npix;  // N * OH * OW
    FastDiv by_ohw;
    // fused int8 form (apps/cpu/relay/result.log:17-20): out = (acc + bias[channel]) * scale
    const int *bias;  // K values or null
    int scale;
    // requantised u8 output (direct kernels, Q8): a second per-channel addend and the right shift
    const int *bias2;
    int shift;
    // direct kernels: 0 = blocked (N, K/16, OH, OW, 16) output; else the output is planar (N, planar, OH, OW),
    // planar <= K channels (the reference's graphs end in this layout_transform: apps/cpu/relay/result.log:25)
    int planar;
  };
  static constexpr int kPitch = 144;               // bytes per pixel row of the scratch
  static constexpr int kScratch = 32 * kPitch;     // per wave
  // LDS bytes the epilogue needs for a tile shape
  template <class T>
  static constexpr int lds_bytes() {
    return (T::NTG / 64) * (kScratch + T::TX * 32 * 4);
  }

  template <class T>
  static __device__ __forceinline__ void store(const Params &p, typename Op::acc_t (&acc)[T::TX][T::TY],
                                               int (&wsx)[T::TX], int (&)[T::TY], int xw0, int yw0, int lane,
                                               int wave, char *lds, bool accumulate) {
    using out_t = typename Op::out_t;
    using out4_t = typename Op::out4_t;
    const int l32 = lane & 31, half = lane >> 5;
    char *scratch = lds + wave * kScratch;
    int *wsb = reinterpret_cast<int *>(lds + (T::NTG / 64) * kScratch) + wave * (T::TX * 32);
    if constexpr (Op::kInt) {
      if (half == 0) {
#pragma unroll
        for (int i = 0; i < T::TX; ++i) {
          const int c = xw0 + i * 32 + l32;
          wsb[i * 32 + l32] = (wsx[i] << 7) + (p.bias != nullptr && c < p.K ? p.bias[c] : 0);
        }
      }
    }
    const int ko_planes = p.K >> 4;
    const int rp = lane >> 2, piece = lane & 3;  // read-back role: pixel row, 16-byte piece
#pragma unroll
    for (int j = 0; j < T::TY; ++j) {
      // the two pixels this lane stores for block column j
      size_t obase[2];
      bool ok[2];
#pragma unroll
      for (int it = 0; it < 2; ++it) {
        const int m = yw0 + j * 32 + it * 16 + rp;
        ok[it] = m < p.npix;
        int n, pix;
        p.by_ohw.divmod(m, n, pix);
        obase[it] = ((size_t)n * ko_planes * p.ohw + pix) * 16 + piece * 4;
      }
#pragma unroll
      for (int i = 0; i < T::TX; ++i) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int cl = i * 32 + 8 * q + 4 * half;  // channel inside the wave's X range
          out4_t v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
          if constexpr (Op::kInt) v = (v + *reinterpret_cast<const v4i *>(wsb + cl)) * p.scale;
          *reinterpret_cast<out4_t *>(scratch + l32 * kPitch + (8 * q + 4 * half) * 4) = v;
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int c = xw0 + i * 32 + h * 16;  // first channel of this 16-channel plane
          if (c >= p.K) continue;
#pragma unroll
          for (int it = 0; it < 2; ++it) {
            const out4_t v = *reinterpret_cast<const out4_t *>(scratch + (it * 16 + rp) * kPitch + h * 64 + piece * 16);
            if (!ok[it]) continue;
            out_t *dst = reinterpret_cast<out_t *>(p.out) + obase[it] + (size_t)(c >> 4) * p.ohw * 16;
            if (accumulate) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                if constexpr (Op::kInt)
                  atomicAdd(dst + e, v[e]);
                else
                  unsafeAtomicAdd(dst + e, v[e]);
              }
            } else {
              store_result(result_buffer(p.out), (u32)((obase[it] + (size_t)(c >> 4) * p.ohw * 16) * sizeof(out_t)), v);
            }
          }
        }
      }
    }
  }
};

}  // namespace unit
