// int8 convolution in NCHW{16,4}c as an implicit GEMM: X operand = weights (rows = output
// channels, read straight from the reference's (K/16, C/cb, KH, KW, cb/4, 16, 4) pre-pack),
// Y operand = output pixels gathered on the fly from the u8 data tensor.
// Included by conv_i8_c16.hip / conv_i8_c4.hip, one translation unit per channel block.
#pragma once
#include "conv_plan.hpp"
#include "epilogues.hpp"

namespace unit {

template <class T, int TAPB, int PF>
int run_conv_i8(const unit_conv_desc *d, const ConvGeom &g0, const void *data, const void *w, void *out, int splits,
                hipStream_t s) {
  using XL = VnniLoader<T::BX, T::BKB, T::NT, 16, PF>;
  using YL = ConvPixelLoader<T::BY, T::BKB, T::NT, TAPB, true, PF>;
  using Epi = ConvEpilogue<OpI8>;
  ConvGeom g = g0;
  const int kbytes = g.ntaps * TAPB;
  const int nk = ceil_div(kbytes, T::BKB);
  g.ntab = nk * T::BKB / TAPB;
  typename XL::Params xp{static_cast<const char *>(w), d->K, kbytes / 4};
  typename YL::Params yp{static_cast<const char *>(data), g};
  typename Epi::Params ep{out, d->K, g.OH * g.OW, g.npix};
  const int gx = ceil_div(d->K, T::BX), gy = ceil_div(g.npix, T::BY);
  if (splits > nk) splits = nk;
  set_variant("i8conv_c%d_x%d_y%d_k%d_w%d_p%d%s_s%d", TAPB, T::BX, T::BY, T::BKB, T::NT / 64, PF, T::FF ? "f" : "", splits);
  return launch_mma<OpI8, T, XL, YL, Epi, WS_X>(xp, yp, ep, nk, gx, gy, gx, splits, out,
                                                (size_t)g.npix * d->K * 4, g.ntab * 8, s,
                                                "unit_conv2d_nchwc_u8s8s32");
}

template <int TAPB>
int run_conv_i8_variant(int variant, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                        void *out, int splits, hipStream_t s) {
#define UNIT_CASE_FF(ID, BX, BY, BKB, WX, WY, PF) \
  case ID:                                        \
    return run_conv_i8<Tile<BX, BY, BKB, WX, WY, true>, TAPB, PF>(d, g, data, w, out, splits, s)
#define UNIT_CASE(ID, BX, BY, BKB, WX, WY, PF) \
  case ID:                                     \
    return run_conv_i8<Tile<BX, BY, BKB, WX, WY>, TAPB, PF>(d, g, data, w, out, splits, s)
  switch (variant) {
    UNIT_CASE(0, 256, 256, 128, 2, 4, 1);
    UNIT_CASE(1, 256, 256, 64, 2, 4, 1);
    UNIT_CASE(2, 128, 256, 128, 2, 4, 1);
    UNIT_CASE(3, 128, 256, 64, 2, 4, 1);
    UNIT_CASE(4, 64, 256, 128, 1, 4, 1);
    UNIT_CASE(5, 64, 256, 64, 1, 4, 1);
    UNIT_CASE(6, 128, 128, 128, 2, 2, 1);
    UNIT_CASE(7, 128, 128, 64, 2, 2, 1);
    UNIT_CASE(8, 256, 128, 128, 2, 2, 1);
    UNIT_CASE(9, 256, 128, 64, 2, 2, 1);
    UNIT_CASE(10, 64, 128, 64, 1, 4, 1);
    UNIT_CASE(11, 64, 64, 64, 2, 2, 1);
    UNIT_CASE(12, 256, 256, 128, 2, 2, 1);
    UNIT_CASE(13, 256, 256, 64, 2, 2, 1);
    UNIT_CASE(14, 128, 64, 128, 2, 2, 1);
    UNIT_CASE(15, 64, 128, 128, 1, 4, 1);
    UNIT_CASE(16, 128, 64, 128, 2, 2, 3);
    UNIT_CASE(17, 64, 128, 128, 1, 4, 3);
    UNIT_CASE(18, 128, 128, 128, 2, 2, 2);
    UNIT_CASE(19, 64, 64, 64, 2, 2, 4);
    UNIT_CASE(20, 64, 256, 64, 1, 4, 2);
    UNIT_CASE(21, 64, 128, 64, 1, 4, 3);
    UNIT_CASE(22, 128, 256, 128, 2, 4, 2);
    UNIT_CASE(23, 128, 64, 128, 2, 2, 2);
    UNIT_CASE(24, 128, 128, 64, 2, 2, 3);
    UNIT_CASE(25, 256, 128, 64, 2, 2, 2);
    UNIT_CASE(26, 64, 32, 128, 2, 1, 2);
    UNIT_CASE(27, 128, 32, 128, 2, 1, 2);
    UNIT_CASE(28, 64, 64, 128, 2, 1, 2);
    UNIT_CASE(29, 64, 32, 64, 2, 1, 3);
    UNIT_CASE(30, 128, 64, 128, 2, 1, 2);
    UNIT_CASE(31, 128, 64, 128, 4, 1, 2);
    UNIT_CASE_FF(32, 128, 64, 128, 2, 2, 2);
    UNIT_CASE_FF(33, 64, 64, 64, 2, 2, 4);
    UNIT_CASE_FF(34, 64, 32, 128, 2, 1, 2);
    UNIT_CASE_FF(35, 128, 128, 128, 2, 2, 2);
    UNIT_CASE_FF(36, 64, 128, 128, 1, 4, 2);
    UNIT_CASE_FF(37, 128, 32, 128, 2, 1, 2);
    UNIT_CASE_FF(38, 64, 64, 128, 2, 2, 2);
    UNIT_CASE_FF(39, 128, 64, 128, 2, 2, 4);
    default:
      return fail(UNIT_E_ARG, "unit_conv2d_nchwc_u8s8s32: unknown kernel variant %d", variant);
  }
#undef UNIT_CASE
#undef UNIT_CASE_FF
}

}  // namespace unit
