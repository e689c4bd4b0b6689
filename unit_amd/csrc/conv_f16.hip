// fp16 convolution NCHW16c x (K/16, C/16, KH, KW, 16 in, 16 out) -> f32 NCHW16c as an implicit
// GEMM: X operand = weights (rows = output channels, transposed while staging), Y operand =
// output pixels gathered on the fly.  Same tile variants and planner as the int8 convolution.
#include "conv_plan.hpp"
#include "epilogues.hpp"

namespace unit {

int conv_geom(const unit_conv_desc *d, int tapb, ConvGeom *g, const char *what);  // abi.hip
int conv_f16_direct(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *a, const void *b,
                    void *out, hipStream_t s);  // conv_direct_f16.hip

namespace {

template <class T, int PF>
int run_conv_f16(const unit_conv_desc *d, const ConvGeom &g0, const void *a, const void *b, void *out,
                 const ConvPlan &plan, hipStream_t s) {
  using XL = KMajorF16Loader<T::BX, T::BKB, T::NTG, PF>;
  using YL = ConvPixelLoader<T::BY, T::BKB, T::NTG, 32, false, PF>;
  using Epi = ConvEpilogue<OpF16>;
  ConvGeom g = g0;
  const int kbytes = g.ntaps * 32;
  const int nk = ceil_div(kbytes, T::BKB);
  g.ntab = nk * T::BKB / 32;
  // weight element (ko, tap, i, o): ((ko * ntaps + tap) * 16 + i) * 16 + o  -> k = tap*16 + i
  typename XL::Params xp{static_cast<const char *>(b), d->K, g.ntaps * 16, 16, (size_t)g.ntaps * 512, 32};
  typename YL::Params yp{static_cast<const char *>(a), g};
  typename Epi::Params ep{out, d->K, g.OH * g.OW, g.npix, g.by_ohw, nullptr, 1, nullptr, 0};
  const int gx = ceil_div(d->K, T::BX), gy = ceil_div(g.npix, T::BY);
  const int panel = plan.panel > 0 && plan.panel < gx ? plan.panel : 0;
  char tail[16] = "";
  if (panel) snprintf(tail, sizeof tail, "_r%d", panel);
  set_variant("f16conv_x%d_y%d_k%d_w%dx%d_p%d%s%s%s", T::BX, T::BY, T::BKB, T::WX, T::WY, PF, T::FF ? "f" : "",
              T::KG == 1 ? "" : (T::KG == 2 ? "_g2" : "_g4"), tail);
  return launch_mma<OpF16, T, XL, YL, Epi, WS_NONE>(xp, yp, ep, nk, gx, gy, panel ? panel : gx, 1, out, 0, g.ntab * 8, s,
                                                    "unit_conv2d_nchw16c_f16f32");
}

int run_conv_f16_variant(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *a,
                         const void *b, void *out, hipStream_t s) {
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D)
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG) \
  case ID:                                                     \
    return run_conv_f16<Tile<BX, BY, BKB, WX, WY, FF, KG>, PF>(d, g, a, b, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "unit_conv2d_nchw16c_f16f32: kernel variant %d not available for this layout", plan.variant);
  }
#undef UNIT_CONV_VARIANT
#undef UNIT_CONV_DIRECT
}

// measured on MI355X by `python -m unit_amd.tune --dtype f16` (key: N*OH*OW, K, C, KH, KW, stride)
const TunedConv kTunedF16[] = {
#include "tuned_conv_f16.inc"
    {0, 0, 0, 0, 0, 0, 0, 0, 0},
};

}  // namespace
}  // namespace unit

extern "C" int unit_conv2d_nchw16c_f16f32(const unit_conv_desc *d, const void *a, const void *b, void *out,
                                          unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv2d_nchw16c_f16f32";
  if (!d || !a || !b || !out) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (d->cb != 16) return fail(UNIT_E_ARG, "%s: cb must be 16 (got %d)", what, d->cb);
  if (d->pt || d->pl || d->pb || d->pr) return fail(UNIT_E_ARG, "%s: the operator has no padding argument; pre-pad the data", what);
  if (d->dh != 1 || d->dw != 1) return fail(UNIT_E_ARG, "%s: dilation must be 1", what);
  size_t in_img, out_img;
  if (const int per = batch_slice(d, (size_t)d->C * 2, (size_t)d->K * 4, &in_img, &out_img))
    return run_batch_slices(d, per, in_img, out_img, a, out, [&](const unit_conv_desc *sd, const void *x, void *y) {
      return unit_conv2d_nchw16c_f16f32(sd, x, b, y, stream);
    });
  ConvGeom g;
  if (int rc = conv_geom(d, 32, &g, what)) return rc;
  if (!fits((size_t)g.npix * d->K * 4)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {a, b, out})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int ntable = (int)(sizeof(kTunedF16) / sizeof(kTunedF16[0])) - 1;
  // no k-splits: fp32 atomics would make the summation order, and so the result, vary run to run
  const ConvPlan p = plan_conv(d, g.npix, g.ntaps * 32, kTunedF16, ntable, false, true, true);
  if (kConvTiles[p.variant].direct) return conv_f16_direct(p, d, g, a, b, out, s);
  return run_conv_f16_variant(p, d, g, a, b, out, s);
}
