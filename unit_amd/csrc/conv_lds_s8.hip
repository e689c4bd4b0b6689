// LDS-shared variants of the fused signed NCHW16c convolution on prepared weights:
// out = (conv(x, w) + bias) * scale, blocked or planar (NCHW) int32 output.
#include "conv_lds_host.hpp"

namespace unit {

int conv_s8_prepared_lds(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                         const char *zero, const int *bias, int scale, void *out, int planar, hipStream_t s) {
  const char *what = planar ? "unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw" : "unit_conv2d_nchwc_s8s8s32_fused_prepared";
  const char *tag = planar ? "s8lds_c16_nchw" : "s8lds_c16";
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)
#define UNIT_CONV_LDS(ID, TX, TY, WX, WY, KG, KS, NST)                                                                    \
  case ID:                                                                                                                \
    return planar ? run_lds<LdsShape<TX, TY, WX, WY, KG, KS, NST>, false, false, true>(what, tag, d, g, data, w, zero, bias, \
                                                                                       scale, out, plan, s, nullptr, 0, planar) \
                  : run_lds<LdsShape<TX, TY, WX, WY, KG, KS, NST>, false>(what, tag, d, g, data, w, zero, bias, scale, out, plan, s);
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
