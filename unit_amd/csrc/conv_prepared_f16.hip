// Direct variants of the fp16 NCHW16c convolution on prepared weights.
#include "conv_direct_host.hpp"

namespace unit {

int conv_f16_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *a, const void *w,
                      void *out, hipStream_t s) {
  const char *what = "unit_conv2d_nchw16c_f16f32_prepared";
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D) \
  case ID:                                  \
    return run_direct<OpF16, DirectShape<TX, TY, KG, D, false>, false, true>(what, "f16prep", d, g, a, w, nullptr, 1, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: unknown kernel variant %d", what, plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
