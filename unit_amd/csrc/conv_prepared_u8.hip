// Direct variants of the u8 x s8 -> i32 NCHW16c convolution on prepared weights.
#include "conv_direct_host.hpp"

namespace unit {

int conv_u8_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                     const int *addend, void *out, hipStream_t s) {
  const char *what = "unit_conv2d_nchwc_u8s8s32_prepared";
  // the fragment that pads an odd tap count is zero, so only real zero padding needs the tap masks
  const bool masked = d->pt || d->pl || d->pb || d->pr;
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)                                                                            \
  case ID:                                                                                                             \
    return masked ? run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, true, true>(what, "i8prep_c16", d, g, data, w,  \
                                                                                    addend, 1, out, plan, s)           \
                  : run_direct<OpI8, DirectShape<TX, TY, KG, D, false>, true, true>(what, "i8prep_c16", d, g, data, w, \
                                                                                     addend, 1, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: unknown kernel variant %d", what, plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
