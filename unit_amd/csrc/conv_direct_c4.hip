// Direct variants of the int8 convolution on 4-channel blocks (the 3-channel stems, 2-D and 3-D) with the
// reference's weight layout (K/16, C/4, [KD,] KH, KW, 1, 16, 4): u8 data (shift) and signed data.
#include "conv_direct_host.hpp"

namespace unit {

// true if a convolution on 4-channel blocks can run on the direct kernels: a window row is one k-step
bool conv_c4_direct_ok(const unit_conv_desc *d) { return d->cb == 4 && d->KW <= 8 && d->KH <= 31 && d->dw == 1; }

int conv_c4_direct(const char *what, const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data,
                   const void *w, const int *bias, int scale, bool shift, void *out, hipStream_t s) {
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)                                                                            \
  case ID:                                                                                                             \
    return shift ? run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, true, false, true>(what, "i8direct_c4", d, g,    \
                                                                                          data, w, bias, scale, out,   \
                                                                                          plan, s)                     \
                 : run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, false, false, true>(what, "s8direct_c4", d, g,   \
                                                                                           data, w, bias, scale, out,  \
                                                                                           plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: kernel variant %d not available for this layout", what, plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
