// int8 convolution kernels for 4-channel input blocks (NCHW4c: the 3-channel network stems).
#include "conv_i8_impl.hpp"

namespace unit {
int conv_i8_c4(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
               void *out, hipStream_t s) {
  return run_conv_i8_variant<4>(plan, d, g, data, w, out, s);
}
}  // namespace unit
