// Direct variants of the u8 x s8 -> i32 NCHW16c convolution.
#include "conv_direct_host.hpp"

namespace unit {

int conv_i8_direct(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                   void *out, hipStream_t s) {
  const char *what = "unit_conv2d_nchwc_u8s8s32";
  if (d->cb != 16 || d->KH * d->KW > 31)
    return fail(UNIT_E_ARG, "%s: kernel variant %d not available for this layout or window", what, plan.variant);
  // Without zero padding every tap of a valid pixel lies inside the image and the kernel without
  // tap masks serves; an odd tap count needs the masks too, for the tap that pads the last k-step.
  const bool masked = d->pt || d->pl || d->pb || d->pr || (g.ntaps & 1);
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)                                                                          \
  case ID:                                                                                                           \
    return masked ? run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, true>(what, "i8direct_c16", d, g, data, w,    \
                                                                              nullptr, 1, out, plan, s)                    \
                  : run_direct<OpI8, DirectShape<TX, TY, KG, D, false>, true>(what, "i8direct_c16", d, g, data, w,   \
                                                                               nullptr, 1, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: unknown kernel variant %d", what, plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
