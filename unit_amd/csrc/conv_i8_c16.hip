// int8 convolution kernels for 16-channel input blocks (NCHW16c).
#include "conv_i8_impl.hpp"

namespace unit {
int conv_i8_c16(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                void *out, hipStream_t s) {
  return run_conv_i8_variant<16>(plan, d, g, data, w, out, s);
}
}  // namespace unit
