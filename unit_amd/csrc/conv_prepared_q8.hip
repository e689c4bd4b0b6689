// Direct variants of the u8 x s8 convolution on prepared weights with requantised u8 output
// (16- and 4-channel input blocks).
#include "conv_direct_host.hpp"

namespace unit {

int conv_q8_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                     const int *addend, const int *bias, int scale, int shift, void *out, hipStream_t s) {
  const char *what = "unit_conv2d_nchwc_u8s8u8_requant_prepared";
  const bool masked = d->pt || d->pl || d->pb || d->pr;
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)                                                                            \
  case ID:                                                                                                             \
    if (d->cb == 4)                                                                                                    \
      return run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, true, true, true, true>(                               \
          what, "q8prep_c4", d, g, data, w, addend, scale, out, plan, s, bias, shift);                                 \
    return masked ? run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, true, true, false, true>(                       \
                        what, "q8prep_c16", d, g, data, w, addend, scale, out, plan, s, bias, shift)                   \
                  : run_direct<OpI8, DirectShape<TX, TY, KG, D, false>, true, true, false, true>(                      \
                        what, "q8prep_c16", d, g, data, w, addend, scale, out, plan, s, bias, shift);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: unknown kernel variant %d", what, plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
