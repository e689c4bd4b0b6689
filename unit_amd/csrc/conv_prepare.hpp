// Prepared convolution weights: the MFMA fragment order the direct kernels read with one 16-byte
// load per lane and k-step (conv_direct.hpp, PREP).
//
//   prepared[kb][s][lane][16 bytes], kb = 32-channel block of K, s = k-step, lane = 0..63:
//     int8, 16-channel blocks: channel kb * 32 + lane % 32, tap 2 s + lane / 32 (taps run (ci, kh, kw)
//           as in the reference's (K/16, C/16, KH, KW, 4, 16, 4) layout), its 16 input channels;
//     int8, 4-channel blocks (K/16, C/4, KH, KW, 1, 16, 4): k-step s = ci * KH + kh is one window row,
//           the lane holds taps kw = 4 (lane / 32) .. + 3 of it, 4 input channels each (KW <= 8);
//     fp16: channel kb * 32 + lane % 32, tap s, input channels 8 (lane / 32) .. + 8;
//   channels past K and the tap that pads an odd tap count are zeros;
//   int8 only, behind the fragments: int32 addend[kb * 32 + c] = 128 * sum of the channel's weights
//   (what a u8 convolution computed on x ^ 0x80 has to add back), then 16 KiB of zeros: the weight fragments
//   that the LDS-shared kernels (conv_lds.hpp) read for k-steps past a k-group's share of the reduction.
#pragma once
#include <cstddef>

namespace unit {

struct PreparedLayout {
  int kblocks, nsteps;
  size_t frag_bytes;    // kblocks * nsteps * 1 KiB
  size_t total_bytes;   // + the addends and the zero region for int8
  size_t zero_off;      // int8: byte offset of the zero region
};
// size of the zero region (a wave-level load reads 1 KiB of it; the size is part of the prepared buffer's layout)
constexpr int kZeroLine = 16384;

inline PreparedLayout prepared_layout(int K, int C, int KH, int KW, int cb, int elem_bytes) {
  PreparedLayout p;
  const int ntaps = (C / cb) * KH * KW;
  p.kblocks = (K + 31) / 32;
  p.nsteps = cb == 4 ? (C / 4) * KH : (elem_bytes == 1 ? (ntaps + 1) / 2 : ntaps);
  p.frag_bytes = (size_t)p.kblocks * p.nsteps * 1024;
  p.zero_off = p.frag_bytes + (size_t)p.kblocks * 32 * 4;
  p.total_bytes = elem_bytes == 1 ? p.zero_off + kZeroLine : p.frag_bytes;
  return p;
}

}  // namespace unit
