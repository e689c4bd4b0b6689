// Direct variants of the fused signed NCHW16c convolution, (conv(s8, s8) + bias) * scale, on
// prepared weights.
#include "conv_direct_host.hpp"

namespace unit {

namespace {
template <int TX, int TY, int KG, int D>
int dispatch(bool masked, int planar, const char *what, const char *tag, const unit_conv_desc *d, const ConvGeom &g,
             const void *data, const void *w, const int *bias, int scale, void *out, const ConvPlan &plan, hipStream_t s) {
  if (planar)  // int32 (N, planar, OH, OW) output
    return masked ? run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, false, true, false, false, true>(
                        what, tag, d, g, data, w, bias, scale, out, plan, s, nullptr, 0, planar)
                  : run_direct<OpI8, DirectShape<TX, TY, KG, D, false>, false, true, false, false, true>(
                        what, tag, d, g, data, w, bias, scale, out, plan, s, nullptr, 0, planar);
  return masked ? run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, false, true>(what, tag, d, g, data, w, bias, scale, out,
                                                                                   plan, s)
                : run_direct<OpI8, DirectShape<TX, TY, KG, D, false>, false, true>(what, tag, d, g, data, w, bias, scale, out,
                                                                                    plan, s);
}
}  // namespace

int conv_s8_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                     const int *bias, int scale, void *out, int planar, hipStream_t s) {
  const char *what = planar ? "unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw" : "unit_conv2d_nchwc_s8s8s32_fused_prepared";
  const char *tag = planar ? "s8prep_c16_nchw" : "s8prep_c16";
  const bool masked = d->pt || d->pl || d->pb || d->pr;
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)                                                                             \
  case ID:                                                                                                              \
    return dispatch<TX, TY, KG, D>(masked, planar, what, tag, d, g, data, w, bias, scale, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: unknown kernel variant %d", what, plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
