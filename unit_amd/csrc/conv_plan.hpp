// Kernel-variant selection for the convolution entry points: a table of measured choices for
// known layer shapes (the analogue of the reference's tuned-schedule tables, python/tensorizer/
// tune.py:20-48, which map (ashape, bshape, strides) to a schedule index read from cpu-tune.log /
// gpu-tune.log), a heuristic for every other shape, and a per-process override.
#pragma once
#include "host.hpp"
#include "loaders.hpp"

namespace unit {

struct TileShape {
  int bx, by, bkb, waves, pf;  // waves per workgroup; pf: stages of global loads in flight
  bool ff;                     // all fragments of a stage read at once (small wave tiles)
  int kg;                      // k-groups sharing the output tile
  bool direct;                 // operands straight from global memory to registers (int8 NCHW16c)
  bool lds;                    // operand tiles shared through LDS by direct loads (prepared int8 NCHW16c weights only)
};

// index = variant id used by the tuning table and UNIT_AMD_CONV_VARIANT (1-based there)
constexpr TileShape kConvTiles[] = {
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG) {BX, BY, BKB, (WX) * (WY) * (KG), PF, FF, KG, false, false},
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D) {(TX) * 32, (TY) * 32, 32, KG, (D) % 16, false, KG, true, false},
#define UNIT_CONV_LDS(ID, TX, TY, WX, WY, KG, KS, NST) \
  {(TX) * (WX) * 32, (TY) * (WY) * 32, 32 * (KS), (WX) * (WY) * (KG), NST, false, KG, false, true},
#include "conv_variants.def"
#undef UNIT_CONV_LDS
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
};
constexpr int kNumConvTiles = sizeof(kConvTiles) / sizeof(kConvTiles[0]);

struct ConvPlan {
  int variant;
  int splits;
  // Channel tiles per panel of the workgroup -> tile walk (0: all of them).  An XCD's workgroups
  // cover whole panels, so 0 makes every XCD read all weights and a slice of the pixels, while
  // a small panel gives each XCD a slice of the weights and all pixels: the better choice is the
  // one that pulls fewer bytes into the 8 L2s, which start cold at every kernel.
  int panel;
};

struct TunedConv {
  int npix, K, C, KH, KW, sh;  // key
  int variant, splits, panel;
};

// Heuristic for shapes the table does not hold, distilled from the tuning runs: output-bound
// layers (few input channels, many pixels) want 64..128-pixel tiles of 64 channels with many
// workgroups in flight; long reductions want the 128-channel tiles with two stages of loads in
// flight; the 256 x 256 tiles only pay when they still give every CU several workgroups.
inline ConvPlan heuristic_plan(int npix, int K, int kbytes, bool allow_split, bool direct_ok, bool strided = false,
                               bool staged_too = false) {
  const bool k128 = kbytes % 128 == 0;
  const auto tiles = [&](int bx, int by) { return (long)ceil_div(K, bx) * ceil_div(npix, by); };
  if (direct_ok) {
    // NCHW16c: the direct kernels won every tuned layer but the widest outputs.  One wave per
    // 64 x 64 tile when the tiles alone fill the SIMDs, else k-groups (4, 8) to put about a
    // thousand waves on the chip; the smallest problems use 64 x 32 (fp16: 32 x 64) tiles.
    const long t64 = tiles(64, 64);
    int v, panel = 0;
    if (allow_split) {  // the int8 operator; distilled from the tuner's choices on cold operands (batch 1 .. 256)
      const int nsteps = kbytes / 32;
      const bool wide = K % 128 == 0;  // 128-channel tiles
      if (t64 < 196)
        v = 60;  // 64 x 32 tiles, four k-groups, six deep
      else if (t64 < 392)
        v = nsteps >= 36 ? 63 : 52;  // 64 x 64, four k-groups: six deep for long reductions, else four
      else if (t64 < 784)
        v = nsteps <= 4 ? 70 : (nsteps <= 8 ? 50 : (nsteps < 72 || !wide ? 52 : 56));
      else if (t64 < 1568)
        v = nsteps <= 4 ? 70 : (nsteps <= 16 ? 71 : 68);  // one wave per tile: 2 / 3 deep at four waves per SIMD, then 6 deep
      else if (t64 < 3136)
        v = nsteps <= 8 ? 70 : (wide ? 54 : 71);  // 128-channel tiles while they still give every SIMD a wave
      else
        v = nsteps <= 36 ? 70 : 68;
      // Eight or more channel tiles: panels of four, so that an XCD's L2 holds a slice of the weights for all its
      // pixels; not when the stride skips input pixels (the data is then the sparse operand), nor when a long
      // reduction already keeps a large problem's weights hot.
      if (K >= 512 && !strided && (nsteps <= 16 || t64 < 784)) panel = 4;
    } else {  // the fp16 operator (a k-step is one tap of 16 channels), same source
      const int nsteps = kbytes / 32;
      const bool wide = K % 128 == 0;
      // Weights in the reference's layout (staged_too): with a reduction of 32 steps or more and enough large tiles
      // the staged kernels, which share both operands through LDS, beat the direct ones (batch 256: 3 x 3 256 -> 256
      // on 14 x 14 in 69 against 122 us; measured gain 5 - 45 % from 98 tiles of 256 x 256 up, a loss below)
      if (staged_too && nsteps >= 32) {
        if (K % 256 == 0 && tiles(256, 256) >= 196) return ConvPlan{0, 1, 0};
        if (wide && tiles(256, 256) >= 98) return ConvPlan{18, 1, 0};
      }
      if (t64 < 196)
        v = 60;
      else if (t64 < 392)
        v = nsteps <= 8 ? 50 : 52;
      else if (t64 < 784)
        v = nsteps <= 8 ? 50 : (nsteps <= 36 || !wide ? 68 : 56);
      else if (t64 < 1568)
        v = nsteps <= 8 ? 65 : (!wide ? 68 : (nsteps <= 36 ? 54 : 55));
      else
        v = nsteps <= 8 ? 50 : (wide ? 54 : 68);
    }
    return ConvPlan{v, 1, panel};
  }
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
  return ConvPlan{v, splits, 0};
}

inline ConvPlan plan_conv(const unit_conv_desc *d, int npix, int kbytes, const TunedConv *table, int ntable,
                          bool allow_split, bool direct_ok, bool staged_too = false, bool lds_ok = false) {
  ConvPlan p = heuristic_plan(npix, d->K, kbytes, allow_split, direct_ok, d->sh * d->sw > 1, staged_too);
  // UNIT_AMD_CONV_NOTABLE=1: heuristic only (the tuner measures it as the baseline)
  if (tuning_override("UNIT_AMD_CONV_NOTABLE") > 0) ntable = 0;
  for (int i = 0; i < ntable; ++i) {
    const TunedConv &e = table[i];
    // the tables were tuned on square strides without dilation; a direct choice needs a window the direct
    // kernels can run, otherwise the heuristic's (staged) choice stands
    if (e.npix == npix && e.K == d->K && e.C == d->C && e.KH == d->KH && e.KW == d->KW && e.sh == d->sh &&
        d->sw == d->sh && d->dh == 1 && d->dw == 1 && (direct_ok || !kConvTiles[e.variant].direct) &&
        (lds_ok || !kConvTiles[e.variant].lds)) {
      p = ConvPlan{e.variant, e.splits, e.panel};
      break;
    }
  }
  // A direct variant whose k-groups park one float tile each can outgrow the LDS on very deep reductions (the tap
  // table follows the tiles): the one-wave six-deep kernel of the same family always fits.
  if (!allow_split && kConvTiles[p.variant].direct && kConvTiles[p.variant].kg > 1) {
    const TileShape &t = kConvTiles[p.variant];
    const long tile = (long)t.bx * t.by * 4 + t.bx * 4, scratch = 32 * 144 + 128;  // DirectShape: TILE + WSUM, kScratch
    if (t.kg * (scratch + tile) + (long)(kbytes / 32) * 8 > kMaxLds) p = ConvPlan{68, 1, p.panel};
  }
  const int ov = tuning_override("UNIT_AMD_CONV_VARIANT"), os = tuning_override("UNIT_AMD_CONV_SPLITK");
  if (ov > 0 && ov <= kNumConvTiles) p.variant = ov - 1;
  if (os > 0) p.splits = os;
  const int op = tuning_override("UNIT_AMD_CONV_PANEL");
  if (op > 0) p.panel = op;
  if (!allow_split) p.splits = 1;
  // the LDS-shared variants exist for prepared weights with 16-channel blocks only: elsewhere their ids run the heuristic's choice
  if (kConvTiles[p.variant].lds && !lds_ok) {
    const ConvPlan h = heuristic_plan(npix, d->K, kbytes, allow_split, direct_ok, d->sh * d->sw > 1, staged_too);
    p.variant = h.variant;
    if (!allow_split) p.splits = 1;
  }
  return p;
}

}  // namespace unit
