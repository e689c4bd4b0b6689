// int8 convolution in NCHW{16,4}c as an implicit GEMM: X operand = weights (rows = output
// channels, read straight from the reference's (K/16, C/cb, KH, KW, cb/4, 16, 4) pre-pack),
// Y operand = output pixels gathered on the fly from the u8 data tensor.
#include "epilogues.hpp"
#include "host.hpp"
#include "loaders.hpp"

namespace unit {

int conv_geom(const unit_conv_desc *d, int tapb, ConvGeom *g, const char *what);  // abi.hip

namespace {

template <class T, int TAPB>
int run_conv(const unit_conv_desc *d, const ConvGeom &g0, const void *data, const void *w, void *out,
             hipStream_t s) {
  using XL = VnniLoader<T::BX, T::BKB, T::NT, 16>;
  using YL = ConvPixelLoader<T::BY, T::BKB, T::NT, TAPB, true>;
  using Epi = ConvEpilogue<OpI8>;
  ConvGeom g = g0;
  const int kbytes = g.ntaps * TAPB;
  const int nk = ceil_div(kbytes, T::BKB);
  g.ntab = nk * T::BKB / TAPB;
  typename XL::Params xp{static_cast<const char *>(w), d->K, kbytes / 4};
  typename YL::Params yp{static_cast<const char *>(data), g};
  typename Epi::Params ep{out, d->K, g.OH * g.OW, g.npix};
  const int gx = ceil_div(d->K, T::BX), gy = ceil_div(g.npix, T::BY);
  set_variant("i8conv_c%d_x%d_y%d_k%d_w%d", TAPB, T::BX, T::BY, T::BKB, T::NT / 64);
  return launch_mma<OpI8, T, XL, YL, Epi, WS_X>(xp, yp, ep, nk, gx, gy, gx, g.ntab * 8, s,
                                                "unit_conv2d_nchwc_u8s8s32");
}

template <int TAPB>
int dispatch(const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w, void *out,
             hipStream_t s) {
  const int kbytes = g.ntaps * TAPB;
  const bool k128 = kbytes % 128 == 0;
  if (d->K % 256 == 0 && g.npix >= 256 * 64) {
    if (k128) return run_conv<Tile<256, 256, 128, 2, 4>, TAPB>(d, g, data, w, out, s);
    return run_conv<Tile<256, 256, 64, 2, 4>, TAPB>(d, g, data, w, out, s);
  }
  if (d->K % 128 == 0 && g.npix >= 256 * 32) {
    if (k128) return run_conv<Tile<128, 256, 128, 2, 4>, TAPB>(d, g, data, w, out, s);
    return run_conv<Tile<128, 256, 64, 2, 4>, TAPB>(d, g, data, w, out, s);
  }
  if (g.npix >= 256 * 32) {
    if (k128) return run_conv<Tile<64, 256, 128, 1, 4>, TAPB>(d, g, data, w, out, s);
    return run_conv<Tile<64, 256, 64, 1, 4>, TAPB>(d, g, data, w, out, s);
  }
  return run_conv<Tile<64, 64, 64, 2, 2>, TAPB>(d, g, data, w, out, s);
}

}  // namespace
}  // namespace unit

extern "C" int unit_conv2d_nchwc_u8s8s32(const unit_conv_desc *d, const void *data, const void *weight,
                                         void *out, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv2d_nchwc_u8s8s32";
  if (!d || !data || !weight || !out) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (d->cb != 16 && d->cb != 4) return fail(UNIT_E_ARG, "%s: cb must be 16 or 4 (got %d)", what, d->cb);
  ConvGeom g;
  if (int rc = conv_geom(d, d->cb, &g, what)) return rc;
  if (!fits((size_t)g.npix * d->K * 4)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return d->cb == 16 ? dispatch<16>(d, g, data, weight, out, s) : dispatch<4>(d, g, data, weight, out, s);
}
