// Direct variants of the int8 convolution on 4-channel blocks (the 3-channel stem) with prepared
// weights: u8 data (shift correction from the prepared addend) and the fused signed form.
#include "conv_direct_host.hpp"

namespace unit {

int conv_c4_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                     const int *addend, int scale, bool shift, void *out, int planar, hipStream_t s) {
  const char *what = shift    ? "unit_conv2d_nchwc_u8s8s32_prepared"
                     : planar ? "unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw"
                              : "unit_conv2d_nchwc_s8s8s32_fused_prepared";
  const char *tag = planar ? "s8prep_c4_nchw" : "s8prep_c4";
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)                                                                            \
  case ID:                                                                                                             \
    if (shift)                                                                                                         \
      return run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, true, true, true>(what, "i8prep_c4", d, g, data, w,    \
                                                                                  addend, 1, out, plan, s);            \
    if (planar)                                                                                                        \
      return run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, false, true, true, false, true>(                       \
          what, tag, d, g, data, w, addend, scale, out, plan, s, nullptr, 0, planar);                                  \
    return run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, false, true, true>(what, tag, d, g, data, w, addend,     \
                                                                                 scale, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: unknown kernel variant %d", what, plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
