// fp16 convolution NCHW16c x (K/16, C/16, KH, KW, 16 in, 16 out) -> f32 NCHW16c as an implicit
// GEMM: X operand = weights (rows = output channels, transposed while staging), Y operand =
// output pixels gathered on the fly.
#include "epilogues.hpp"
#include "host.hpp"
#include "loaders.hpp"

namespace unit {

int conv_geom(const unit_conv_desc *d, int tapb, ConvGeom *g, const char *what);  // abi.hip

namespace {

template <class T>
int run_conv_f16(const unit_conv_desc *d, const ConvGeom &g0, const void *a, const void *b, void *out,
                 hipStream_t s) {
  using XL = KMajorF16Loader<T::BX, T::BKB, T::NT>;
  using YL = ConvPixelLoader<T::BY, T::BKB, T::NT, 32, false>;
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
  set_variant("f16conv_x%d_y%d_k%d_w%d", T::BX, T::BY, T::BKB, T::NT / 64);
  return launch_mma<OpF16, T, XL, YL, Epi, WS_NONE>(xp, yp, ep, nk, gx, gy, gx, 1, out, 0, g.ntab * 8, s,
                                                    "unit_conv2d_nchw16c_f16f32");
}

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
  if (d->K % 256 == 0 && g.npix >= 256 * 64) return run_conv_f16<Tile<256, 256, 128, 2, 4>>(d, g, a, b, out, s);
  if (d->K % 128 == 0 && g.npix >= 256 * 32) return run_conv_f16<Tile<128, 256, 128, 2, 4>>(d, g, a, b, out, s);
  if (g.npix >= 256 * 32) return run_conv_f16<Tile<64, 256, 128, 1, 4>>(d, g, a, b, out, s);
  return run_conv_f16<Tile<64, 64, 64, 2, 2>>(d, g, a, b, out, s);
}
