// C-ABI entry of the int8 convolution: validates, plans (tile variant + k-splits) and dispatches.
#include "conv_plan.hpp"

namespace unit {

int conv_geom(const unit_conv_desc *d, int tapb, ConvGeom *g, const char *what);  // abi.hip
int conv_i8_c16(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                void *out, hipStream_t s);
int conv_i8_direct(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                   void *out, hipStream_t s);
bool conv_c4_direct_ok(const unit_conv_desc *d);  // conv_direct_c4.hip
int conv_c4_direct(const char *what, const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data,
                   const void *w, const int *bias, int scale, bool shift, void *out, hipStream_t s);
int conv_i8_c4(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
               void *out, hipStream_t s);

namespace {
// measured on MI355X by `python -m unit_amd.tune` (key: N*OH*OW, K, C, KH, KW, stride)
const TunedConv kTunedI8[] = {
#include "tuned_conv_i8.inc"
    {0, 0, 0, 0, 0, 0, 0, 0, 0},
};
}  // namespace

// the tuned choices also serve the fused signed operator (same shapes, same kernels)
const TunedConv *tuned_conv_i8(int *n) {
  *n = (int)(sizeof(kTunedI8) / sizeof(kTunedI8[0])) - 1;
  return kTunedI8;
}
}  // namespace unit

extern "C" int unit_conv_variant_count(void) { return unit::kNumConvTiles; }

extern "C" int unit_conv_variant_is_direct(int32_t variant) {
  if (variant < 0 || variant >= unit::kNumConvTiles) return -1;
  return unit::kConvTiles[variant].lds ? 2 : (unit::kConvTiles[variant].direct ? 1 : 0);
}

extern "C" int unit_conv2d_nchwc_u8s8s32(const unit_conv_desc *d, const void *data, const void *weight,
                                         void *out, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv2d_nchwc_u8s8s32";
  if (!d || !data || !weight || !out) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (d->cb != 16 && d->cb != 4) return fail(UNIT_E_ARG, "%s: cb must be 16 or 4 (got %d)", what, d->cb);
  size_t in_img, out_img;
  if (const int per = batch_slice(d, (size_t)d->C, (size_t)d->K * 4, &in_img, &out_img))
    return run_batch_slices(d, per, in_img, out_img, data, out, [&](const unit_conv_desc *sd, const void *x, void *y) {
      return unit_conv2d_nchwc_u8s8s32(sd, x, weight, y, stream);
    });
  ConvGeom g;
  if (int rc = conv_geom(d, d->cb, &g, what)) return rc;
  if (!fits((size_t)g.npix * d->K * 4)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {data, weight, out})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int ntable = (int)(sizeof(kTunedI8) / sizeof(kTunedI8[0])) - 1;
  const bool direct_ok = d->cb == 16 ? d->KH * d->KW <= 31 : conv_c4_direct_ok(d);
  const ConvPlan p = plan_conv(d, g.npix, g.ntaps * d->cb, kTunedI8, ntable, true, direct_ok);
  if (kConvTiles[p.variant].direct) {
    if (!direct_ok) return fail(UNIT_E_ARG, "%s: kernel variant %d not available for this layout or window", what, p.variant);
    return d->cb == 16 ? conv_i8_direct(p, d, g, data, weight, out, s)
                       : conv_c4_direct(what, p, d, g, data, weight, nullptr, 1, true, out, s);
  }
  return d->cb == 16 ? conv_i8_c16(p, d, g, data, weight, out, s) : conv_i8_c4(p, d, g, data, weight, out, s);
}
