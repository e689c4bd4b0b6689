// int8 convolution in NCHW{16,4}c as an implicit GEMM: X operand = weights (rows = output
// channels, read straight from the reference's (K/16, C/cb, KH, KW, cb/4, 16, 4) pre-pack),
// Y operand = output pixels gathered on the fly from the u8 data tensor.
// Included by conv_i8_c16.hip / conv_i8_c4.hip, one translation unit per channel block.
#pragma once
#include "conv_plan.hpp"
#include "epilogues.hpp"

namespace unit {

// SIGNED: the data is s8 (the reference's fused form, apps/cpu/relay/result.log:3-26): no shift to
// s8 while staging, no weight sums; bias and scale are applied by the epilogue.
template <class T, int TAPB, int PF, bool SIGNED = false>
int run_conv_i8(const unit_conv_desc *d, const ConvGeom &g0, const void *data, const void *w, void *out,
                const ConvPlan &plan, hipStream_t s, const int *bias = nullptr, int scale = 1) {
  using XL = VnniLoader<T::BX, T::BKB, T::NTG, 16, PF>;
  using YL = ConvPixelLoader<T::BY, T::BKB, T::NTG, TAPB, !SIGNED, PF>;
  using Epi = ConvEpilogue<OpI8>;
  ConvGeom g = g0;
  const int kbytes = g.ntaps * TAPB;
  const int nk = ceil_div(kbytes, T::BKB);
  g.ntab = nk * T::BKB / TAPB;
  typename XL::Params xp{static_cast<const char *>(w), d->K, kbytes / 4};
  typename YL::Params yp{static_cast<const char *>(data), g};
  typename Epi::Params ep{out, d->K, g.OH * g.OW, g.npix, g.by_ohw, bias, scale, nullptr, 0};
  const char *what = SIGNED ? "unit_conv2d_nchwc_s8s8s32_fused" : "unit_conv2d_nchwc_u8s8s32";
  const int gx = ceil_div(d->K, T::BX), gy = ceil_div(g.npix, T::BY);
  const int splits = plan.splits > nk ? nk : plan.splits;
  const int panel = plan.panel > 0 && plan.panel < gx ? plan.panel : 0;
  char tail[16] = "";
  if (panel) snprintf(tail, sizeof tail, "_r%d", panel);
  set_variant("%s_c%d_x%d_y%d_k%d_w%dx%d_p%d%s%s%s_s%d", SIGNED ? "s8conv" : "i8conv", TAPB, T::BX, T::BY, T::BKB, T::WX, T::WY, PF, T::FF ? "f" : "",
              T::KG == 1 ? "" : (T::KG == 2 ? "_g2" : "_g4"), tail, splits);
  return launch_mma<OpI8, T, XL, YL, Epi, SIGNED ? WS_NONE : WS_X>(xp, yp, ep, nk, gx, gy, panel ? panel : gx, splits,
                                                                   out, (size_t)g.npix * d->K * 4, g.ntab * 8, s, what);
}

template <int TAPB>
int run_conv_i8_variant(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data,
                        const void *w, void *out, hipStream_t s) {
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG) \
  case ID:                                                     \
    return run_conv_i8<Tile<BX, BY, BKB, WX, WY, FF, KG>, TAPB, PF>(d, g, data, w, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "unit_conv2d_nchwc_u8s8s32: kernel variant %d not available for this layout", plan.variant);
  }
#undef UNIT_CONV_VARIANT
#undef UNIT_CONV_DIRECT
}

}  // namespace unit
