// LDS-shared variants of the fp16 NCHW16c convolution on prepared weights.
#include "conv_lds_host.hpp"

namespace unit {

int conv_f16_prepared_lds(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *a, const void *w,
                          void *out, hipStream_t s) {
  const char *what = "unit_conv2d_nchw16c_f16f32_prepared";
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)
#define UNIT_CONV_LDS(ID, TX, TY, WX, WY, KG, KS, NST)                                                                  \
  case ID:                                                                                                             \
    return run_lds<LdsShape<TX, TY, WX, WY, KG, KS, NST>, false, false, false, OpF16>(what, "f16lds", d, g, a, w, nullptr, \
                                                                                      nullptr, 1, out, plan, s);
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
