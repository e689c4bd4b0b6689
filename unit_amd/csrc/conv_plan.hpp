// Kernel-variant selection for the convolution entry points: a table of measured choices for
// known layer shapes (the analogue of the reference's tuned-schedule tables, python/tensorizer/
// tune.py:20-48, which map (ashape, bshape, strides) to a schedule index read from cpu-tune.log /
// gpu-tune.log), a heuristic for every other shape, and a per-process override.
#pragma once
#include "host.hpp"
#include "loaders.hpp"

namespace unit {

struct TileShape {
  int bx, by, bkb, waves, pf;  // pf: stages of global loads in flight
  bool ff = false;             // all fragments of a stage read at once (small wave tiles)
};

// index = variant id used by the tuning table and UNIT_AMD_CONV_VARIANT (1-based there)
constexpr TileShape kConvTiles[] = {
    {256, 256, 128, 8, 1},  // 0
    {256, 256, 64, 8, 1},   // 1
    {128, 256, 128, 8, 1},  // 2
    {128, 256, 64, 8, 1},   // 3
    {64, 256, 128, 4, 1},   // 4
    {64, 256, 64, 4, 1},    // 5
    {128, 128, 128, 4, 1},  // 6
    {128, 128, 64, 4, 1},   // 7
    {256, 128, 128, 4, 1},  // 8
    {256, 128, 64, 4, 1},   // 9
    {64, 128, 64, 4, 1},    // 10
    {64, 64, 64, 4, 1},     // 11
    {256, 256, 128, 4, 1},  // 12
    {256, 256, 64, 4, 1},   // 13
    {128, 64, 128, 4, 1},   // 14
    {64, 128, 128, 4, 1},   // 15
    {128, 64, 128, 4, 3},   // 16
    {64, 128, 128, 4, 3},   // 17
    {128, 128, 128, 4, 2},  // 18
    {64, 64, 64, 4, 4},     // 19
    {64, 256, 64, 4, 2},    // 20
    {64, 128, 64, 4, 3},    // 21
    {128, 256, 128, 8, 2},  // 22
    {128, 64, 128, 4, 2},   // 23
    {128, 128, 64, 4, 3},   // 24
    {256, 128, 64, 4, 2},   // 25
    {64, 32, 128, 2, 2},   // 26
    {128, 32, 128, 2, 2},   // 27
    {64, 64, 128, 2, 2},   // 28
    {64, 32, 64, 2, 3},   // 29
    {128, 64, 128, 2, 2},   // 30
    {128, 64, 128, 4, 2},   // 31
    {128, 64, 128, 4, 2, true},   // 32
    {64, 64, 64, 4, 4, true},   // 33
    {64, 32, 128, 2, 2, true},   // 34
    {128, 128, 128, 4, 2, true},   // 35
    {64, 128, 128, 4, 2, true},   // 36
    {128, 32, 128, 2, 2, true},   // 37
    {64, 64, 128, 4, 2, true},   // 38
    {128, 64, 128, 4, 4, true},   // 39
};
constexpr int kNumConvTiles = sizeof(kConvTiles) / sizeof(kConvTiles[0]);

struct ConvPlan {
  int variant;
  int splits;
};

struct TunedConv {
  int npix, K, C, KH, KW, sh;  // key
  int variant, splits;
};

// Heuristic for shapes the table does not hold, distilled from the tuning runs: output-bound
// layers (few input channels, many pixels) want 64..128-pixel tiles of 64 channels with many
// workgroups in flight; long reductions want the 128-channel tiles with two stages of loads in
// flight; the 256 x 256 tiles only pay when they still give every CU several workgroups.
inline ConvPlan heuristic_plan(int npix, int K, int kbytes, bool allow_split) {
  const bool k128 = kbytes % 128 == 0;
  const auto tiles = [&](int bx, int by) { return (long)ceil_div(K, bx) * ceil_div(npix, by); };
  int v;
  if (K % 128 != 0) {  // 64-channel tiles
    if (kbytes <= 64 || !k128)
      v = tiles(64, 256) >= 1024 ? 20 : (tiles(64, 128) >= 512 ? 10 : 19);
    else
      v = tiles(64, 256) >= 1024 ? 4 : (tiles(64, 128) >= 512 ? 17 : 19);
  } else if (!k128) {  // reduction is an odd number of 64-byte stages
    v = (K % 256 == 0 && tiles(256, 256) >= 512) ? 1 : (tiles(128, 256) >= 512 ? 3 : (tiles(128, 128) >= 256 ? 24 : 19));
  } else {
    v = (K % 256 == 0 && tiles(256, 256) >= 512) ? 0 : (tiles(128, 256) >= 512 ? 2 : (tiles(128, 128) >= 384 ? 18 : 23));
  }
  // k-splits accumulate with device-scope atomics, which this part executes at the memory side
  // (each XCD has its own L2): they only pay when the output is tiny and the reduction long
  // (batch-1 layers with a handful of tiles)
  int splits = 1;
  if (allow_split) {
    const TileShape &t = kConvTiles[v];
    const long nt = tiles(t.bx, t.by);
    const int nk = ceil_div(kbytes, t.bkb);
    while (nt * splits < 96 && nk / (splits * 2) >= 4 && splits < 8) splits *= 2;
  }
  return ConvPlan{v, splits};
}

inline ConvPlan plan_conv(const unit_conv_desc *d, int npix, int kbytes, const TunedConv *table, int ntable,
                          bool allow_split) {
  ConvPlan p = heuristic_plan(npix, d->K, kbytes, allow_split);
  for (int i = 0; i < ntable; ++i) {
    const TunedConv &e = table[i];
    if (e.npix == npix && e.K == d->K && e.C == d->C && e.KH == d->KH && e.KW == d->KW && e.sh == d->sh) {
      p = ConvPlan{e.variant, e.splits};
      break;
    }
  }
  const int ov = tuning_override("UNIT_AMD_CONV_VARIANT"), os = tuning_override("UNIT_AMD_CONV_SPLITK");
  if (ov > 0 && ov <= kNumConvTiles) p.variant = ov - 1;
  if (os > 0) p.splits = os;
  if (!allow_split) p.splits = 1;
  return p;
}

}  // namespace unit
