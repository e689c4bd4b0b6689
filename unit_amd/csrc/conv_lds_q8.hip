// LDS-shared variants of the u8 x s8 NCHW16c convolution with requantised u8 output, on prepared weights.
#include "conv_lds_host.hpp"

namespace unit {

int conv_q8_prepared_lds(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                         const char *zero, const int *addend, const int *bias, int scale, int shift, void *out,
                         hipStream_t s) {
  const char *what = "unit_conv2d_nchwc_u8s8u8_requant_prepared";
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)
#define UNIT_CONV_LDS(ID, TX, TY, WX, WY, KG, KS, NST)                                                              \
  case ID:                                                                                                          \
    return run_lds<LdsShape<TX, TY, WX, WY, KG, KS, NST>, true, true>(what, "q8lds_c16", d, g, data, w, zero, addend, \
                                                                      scale, out, plan, s, bias, shift);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: kernel variant %d does not stage its operands in LDS", what, plan.variant);
  }
#undef UNIT_CONV_LDS
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
