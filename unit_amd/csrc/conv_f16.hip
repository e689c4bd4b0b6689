// fp16 convolution NCHW16c x (K/16, C/16, KH, KW, 16 in, 16 out) -> f32 NCHW16c as an implicit
// GEMM: X operand = weights (rows = output channels, transposed while staging), Y operand =
// output pixels gathered on the fly.  Same tile variants and planner as the int8 convolution.
#include "conv_plan.hpp"
#include "epilogues.hpp"

namespace unit {

int conv_geom(const unit_conv_desc *d, int tapb, ConvGeom *g, const char *what);  // abi.hip

namespace {

template <class T, int PF>
int run_conv_f16(const unit_conv_desc *d, const ConvGeom &g0, const void *a, const void *b, void *out,
                 hipStream_t s) {
  using XL = KMajorF16Loader<T::BX, T::BKB, T::NT, PF>;
  using YL = ConvPixelLoader<T::BY, T::BKB, T::NT, 32, false, PF>;
  using Epi = ConvEpilogue<OpF16>;
  ConvGeom g = g0;
  const int kbytes = g.ntaps * 32;
  const int nk = ceil_div(kbytes, T::BKB);
  g.ntab = nk * T::BKB / 32;
  // weight element (ko, tap, i, o): ((ko * ntaps + tap) * 16 + i) * 16 + o  -> k = tap*16 + i
  typename XL::Params xp{static_cast<const char *>(b), d->K, g.ntaps * 16, 16, (size_t)g.ntaps * 512, 32};
  typename YL::Params yp{static_cast<const char *>(a), g};
  typename Epi::Params ep{out, d->K, g.OH * g.OW, g.npix};
  const int gx = ceil_div(d->K, T::BX), gy = ceil_div(g.npix, T::BY);
  set_variant("f16conv_x%d_y%d_k%d_w%d_p%d%s", T::BX, T::BY, T::BKB, T::NT / 64, PF, T::FF ? "f" : "");
  return launch_mma<OpF16, T, XL, YL, Epi, WS_NONE>(xp, yp, ep, nk, gx, gy, gx, 1, out, 0, g.ntab * 8, s,
                                                    "unit_conv2d_nchw16c_f16f32");
}

int run_conv_f16_variant(int variant, const unit_conv_desc *d, const ConvGeom &g, const void *a, const void *b,
                         void *out, hipStream_t s) {
#define UNIT_CASE_FF(ID, BX, BY, BKB, WX, WY, PF) \
  case ID:                                        \
    return run_conv_f16<Tile<BX, BY, BKB, WX, WY, true>, PF>(d, g, a, b, out, s)
#define UNIT_CASE(ID, BX, BY, BKB, WX, WY, PF) \
  case ID:                                     \
    return run_conv_f16<Tile<BX, BY, BKB, WX, WY>, PF>(d, g, a, b, out, s)
  switch (variant) {
    UNIT_CASE(0, 256, 256, 128, 2, 4, 1);
    UNIT_CASE(1, 256, 256, 64, 2, 4, 1);
    UNIT_CASE(2, 128, 256, 128, 2, 4, 1);
    UNIT_CASE(3, 128, 256, 64, 2, 4, 1);
    UNIT_CASE(4, 64, 256, 128, 1, 4, 1);
    UNIT_CASE(5, 64, 256, 64, 1, 4, 1);
    UNIT_CASE(6, 128, 128, 128, 2, 2, 1);
    UNIT_CASE(7, 128, 128, 64, 2, 2, 1);
    UNIT_CASE(8, 256, 128, 128, 2, 2, 1);
    UNIT_CASE(9, 256, 128, 64, 2, 2, 1);
    UNIT_CASE(10, 64, 128, 64, 1, 4, 1);
    UNIT_CASE(11, 64, 64, 64, 2, 2, 1);
    UNIT_CASE(12, 256, 256, 128, 2, 2, 1);
    UNIT_CASE(13, 256, 256, 64, 2, 2, 1);
    UNIT_CASE(14, 128, 64, 128, 2, 2, 1);
    UNIT_CASE(15, 64, 128, 128, 1, 4, 1);
    UNIT_CASE(16, 128, 64, 128, 2, 2, 3);
    UNIT_CASE(17, 64, 128, 128, 1, 4, 3);
    UNIT_CASE(18, 128, 128, 128, 2, 2, 2);
    UNIT_CASE(19, 64, 64, 64, 2, 2, 4);
    UNIT_CASE(20, 64, 256, 64, 1, 4, 2);
    UNIT_CASE(21, 64, 128, 64, 1, 4, 3);
    UNIT_CASE(22, 128, 256, 128, 2, 4, 2);
    UNIT_CASE(23, 128, 64, 128, 2, 2, 2);
    UNIT_CASE(24, 128, 128, 64, 2, 2, 3);
    UNIT_CASE(25, 256, 128, 64, 2, 2, 2);
    UNIT_CASE(26, 64, 32, 128, 2, 1, 2);
    UNIT_CASE(27, 128, 32, 128, 2, 1, 2);
    UNIT_CASE(28, 64, 64, 128, 2, 1, 2);
    UNIT_CASE(29, 64, 32, 64, 2, 1, 3);
    UNIT_CASE(30, 128, 64, 128, 2, 1, 2);
    UNIT_CASE(31, 128, 64, 128, 4, 1, 2);
    UNIT_CASE_FF(32, 128, 64, 128, 2, 2, 2);
    UNIT_CASE_FF(33, 64, 64, 64, 2, 2, 4);
    UNIT_CASE_FF(34, 64, 32, 128, 2, 1, 2);
    UNIT_CASE_FF(35, 128, 128, 128, 2, 2, 2);
    UNIT_CASE_FF(36, 64, 128, 128, 1, 4, 2);
    UNIT_CASE_FF(37, 128, 32, 128, 2, 1, 2);
    UNIT_CASE_FF(38, 64, 64, 128, 2, 2, 2);
    UNIT_CASE_FF(39, 128, 64, 128, 2, 2, 4);
    default:
      return fail(UNIT_E_ARG, "unit_conv2d_nchw16c_f16f32: unknown kernel variant %d", variant);
  }
#undef UNIT_CASE
#undef UNIT_CASE_FF
}

// measured on MI355X by `python -m unit_amd.tune --dtype f16` (key: N*OH*OW, K, C, KH, KW, stride)
const TunedConv kTunedF16[] = {
#include "tuned_conv_f16.inc"
    {0, 0, 0, 0, 0, 0, 0, 0},
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
  ConvGeom g;
  if (int rc = conv_geom(d, 32, &g, what)) return rc;
  if (!fits((size_t)g.npix * d->K * 4)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int ntable = (int)(sizeof(kTunedF16) / sizeof(kTunedF16[0])) - 1;
  // no k-splits: fp32 atomics would make the summation order, and so the result, vary run to run
  const ConvPlan p = plan_conv(d, g.npix, g.ntaps * 32, kTunedF16, ntable, false);
  return run_conv_f16_variant(p.variant, d, g, a, b, out, s);
}
