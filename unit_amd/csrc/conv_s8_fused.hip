// C-ABI entry and kernels of the fused signed int8 convolution
//   out = (sum x_s8 * w + bias[k]) * scale
// = the reference's fused_nn_contrib_conv2d_NCHWc_subtract_add_multiply on x + 128
// (apps/cpu/relay/result.log:3-26,35).  NCHW16c with windows of up to 31 positions and NCHW4c with
// rows of up to 8 taps run on the direct kernels; everything else on two staged tile shapes.
#include "conv_direct_host.hpp"
#include "conv_i8_impl.hpp"

namespace unit {

int conv_geom(const unit_conv_desc *d, int tapb, ConvGeom *g, const char *what);  // abi.hip
const TunedConv *tuned_conv_i8(int *n);                                             // conv_i8.hip
bool conv_c4_direct_ok(const unit_conv_desc *d);                                    // conv_direct_c4.hip
int conv_c4_direct(const char *what, const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data,
                   const void *w, const int *bias, int scale, bool shift, void *out, hipStream_t s);

// direct kernels on signed data; `what` names the entry point in messages (also used by the 3-D operator)
int conv_s8_direct(const char *kWhat, const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data,
                   const void *w, const int *bias, int scale, void *out, hipStream_t s) {
  // an odd tap count needs the tap masks for the tap that pads the last k-step
  const bool masked = !g.nopad || (g.ntaps & 1);
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)                                                                          \
  case ID:                                                                                                           \
    return masked ? run_direct<OpI8, DirectShape<TX, TY, KG, D, true>, false>(kWhat, "s8direct_c16", d, g, data, w,  \
                                                                               bias, scale, out, plan, s)            \
                  : run_direct<OpI8, DirectShape<TX, TY, KG, D, false>, false>(kWhat, "s8direct_c16", d, g, data, w, \
                                                                                bias, scale, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "%s: kernel variant %d not available for this layout", kWhat, plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

namespace {

const char *kWhat = "unit_conv2d_nchwc_s8s8s32_fused";

template <int TAPB>
int staged_s8(const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w, const int *bias, int scale,
              void *out, hipStream_t s) {
  // many output tiles: 64 x 128 tiles of 64-byte stages; few: 64 x 64 with four stages of loads in flight
  const ConvPlan plan{0, 1, 0};  // no k-splits: the bias is added once
  if ((long)ceil_div(d->K, 64) * ceil_div(g.npix, 128) >= 512)
    return run_conv_i8<Tile<64, 128, 64, 1, 4>, TAPB, 1, true>(d, g, data, w, out, plan, s, bias, scale);
  return run_conv_i8<Tile<64, 64, 64, 2, 2>, TAPB, 4, true>(d, g, data, w, out, plan, s, bias, scale);
}

}  // namespace
}  // namespace unit

extern "C" int unit_conv2d_nchwc_s8s8s32_fused(const unit_conv_desc *d, const void *data, const void *weight,
                                               const int32_t *bias, int32_t scale, void *out, unit_stream_t stream) {
  using namespace unit;
  if (!d || !data || !weight || !out) return fail(UNIT_E_ARG, "%s: null pointer", kWhat);
  if (d->cb != 16 && d->cb != 4) return fail(UNIT_E_ARG, "%s: cb must be 16 or 4 (got %d)", kWhat, d->cb);
  size_t in_img, out_img;
  if (const int per = batch_slice(d, (size_t)d->C, (size_t)d->K * 4, &in_img, &out_img))
    return run_batch_slices(d, per, in_img, out_img, data, out, [&](const unit_conv_desc *sd, const void *x, void *y) {
      return unit_conv2d_nchwc_s8s8s32_fused(sd, x, weight, bias, scale, y, stream);
    });
  ConvGeom g;
  if (int rc = conv_geom(d, d->cb, &g, kWhat)) return rc;
  if (!fits((size_t)g.npix * d->K * 4)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", kWhat);
  if (int rc = check_aligned(kWhat, {data, weight, out})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (d->cb == 16 ? d->KH * d->KW <= 31 : conv_c4_direct_ok(d)) {
    // same shapes, same kernels as the unsigned operator minus shift and weight sums: its plan serves
    int ntable = 0;
    const TunedConv *table = tuned_conv_i8(&ntable);
    ConvPlan p = plan_conv(d, g.npix, g.ntaps * d->cb, table, ntable, true, true);
    if (!kConvTiles[p.variant].direct) p = heuristic_plan(g.npix, d->K, g.ntaps * d->cb, true, true, d->sh * d->sw > 1);
    p.splits = 1;
    if (d->cb == 4) return conv_c4_direct(kWhat, p, d, g, data, weight, bias, scale, false, out, s);
    return conv_s8_direct(kWhat, p, d, g, data, weight, bias, scale, out, s);
  }
  return d->cb == 16 ? staged_s8<16>(d, g, data, weight, bias, scale, out, s)
                     : staged_s8<4>(d, g, data, weight, bias, scale, out, s);
}
