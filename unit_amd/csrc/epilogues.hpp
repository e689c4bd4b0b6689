// Accumulator write-back for mma_kernel.
#pragma once
#include "mma_core.hpp"

namespace unit {

// Row-major C (M, N): X rows are m, Y rows are n.  A lane holds one n (l % 32) and 16 m values,
// so each store instruction writes two 128-byte row segments.  For int8 the weight is the Y
// operand: out = acc + 128 * sum_k w[n][k].
template <class Op, bool OUT_F16>
struct GemmEpilogue {
  struct Params {
    void *c;
    int M, N;
  };
  template <class T>
  static __device__ __forceinline__ void store(const Params &p, typename Op::acc_t (&acc)[T::TX][T::TY],
                                               int (&)[T::TX], int (&wsy)[T::TY], int xw0, int yw0, int lane,
                                               int, char *) {
    const int l32 = lane & 31, half = lane >> 5;
#pragma unroll
    for (int j = 0; j < T::TY; ++j) {
      const int n = yw0 + j * 32 + l32;
      if (n >= p.N) continue;
#pragma unroll
      for (int i = 0; i < T::TX; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = xw0 + i * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
          if (m >= p.M) continue;
          const size_t idx = (size_t)m * p.N + n;
          if constexpr (Op::kInt) {
            reinterpret_cast<int *>(p.c)[idx] = acc[i][j][r] + (wsy[j] << 7);
          } else if constexpr (OUT_F16) {
            reinterpret_cast<_Float16 *>(p.c)[idx] = (_Float16)acc[i][j][r];
          } else {
            reinterpret_cast<float *>(p.c)[idx] = acc[i][j][r];
          }
        }
    }
  }
};

// Convolution output (N, K/16, OH, OW, 16), 4-byte elements: X rows are output channels, Y rows
// are output pixels.  A lane holds one pixel and, per register quad, 4 consecutive channels ->
// one 16-byte store; the two register quads q, q+1 of the two lane halves fill a pixel's
// 64-byte channel block.  For int8 the weight is the X operand; its per-channel sums live in
// other lanes, so they go through LDS once.
template <class Op>
struct ConvEpilogue {
  struct Params {
    void *out;
    int K;     // output channels (multiple of 16)
    int ohw;   // OH * OW
    int npix;  // N * OH * OW
  };
  template <class T>
  static __device__ __forceinline__ void store(const Params &p, typename Op::acc_t (&acc)[T::TX][T::TY],
                                               int (&wsx)[T::TX], int (&)[T::TY], int xw0, int yw0, int lane,
                                               int wave, char *lds) {
    const int l32 = lane & 31, half = lane >> 5;
    int *wsb = reinterpret_cast<int *>(lds) + wave * (T::TX * 32);
    if constexpr (Op::kInt) {
      // the K loop ended with a workgroup barrier: the tile buffers are free
      if (half == 0) {
#pragma unroll
        for (int i = 0; i < T::TX; ++i) wsb[i * 32 + l32] = wsx[i] << 7;
      }
      __syncthreads();
    }
    const int ko_planes = p.K >> 4;
#pragma unroll
    for (int j = 0; j < T::TY; ++j) {
      const int m = yw0 + j * 32 + l32;
      if (m >= p.npix) continue;
      const int n = m / p.ohw, pix = m - n * p.ohw;
      typename Op::out_t *obase =
          reinterpret_cast<typename Op::out_t *>(p.out) + ((size_t)n * ko_planes * p.ohw + pix) * 16;
#pragma unroll
      for (int i = 0; i < T::TX; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int cl = i * 32 + 8 * q + 4 * half;  // channel inside the wave's X range
          const int c = xw0 + cl;
          if (c >= p.K) continue;
          typename Op::out4_t v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                   acc[i][j][4 * q + 3]};
          if constexpr (Op::kInt) v += *reinterpret_cast<const v4i *>(wsb + cl);
          *reinterpret_cast<typename Op::out4_t *>(obase + (size_t)(c >> 4) * p.ohw * 16 + (c & 15)) = v;
        }
    }
  }
};

}  // namespace unit
