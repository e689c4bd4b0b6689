// C-ABI entry of the 3-D signed int8 convolution (apps/cpu/kernel/conv3d.py:39-64): geometry with a
// depth dimension on the direct kernels.  As in that file the channel block is 16 when C is a
// multiple of 16 and 4 otherwise (its 3 -> 4 channel, 7 x 7 x 7 workload).
#include "conv_direct_host.hpp"

namespace unit {

int conv_s8_direct(const char *what, const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data,
                   const void *w, const int *bias, int scale, void *out, hipStream_t s);  // conv_s8_fused.hip
int conv_c4_direct(const char *what, const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data,
                   const void *w, const int *bias, int scale, bool shift, void *out, hipStream_t s);  // conv_direct_c4.hip

}  // namespace unit

extern "C" int unit_conv3d_ncdhwc_s8s8s32(const unit_conv3d_desc *d, const void *data, const void *weight, void *out,
                                          unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv3d_ncdhwc_s8s8s32";
  if (!d || !data || !weight || !out) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (d->N <= 0 || d->C <= 0 || d->D <= 0 || d->H <= 0 || d->W <= 0 || d->K <= 0 || d->KD <= 0 || d->KH <= 0 ||
      d->KW <= 0 || d->stride <= 0)
    return fail(UNIT_E_ARG, "%s: sizes and stride must be positive", what);
  if (d->C % 4 || d->K % 16) return fail(UNIT_E_ARG, "%s: C (%d) must be a multiple of 4 and K (%d) of 16", what, d->C, d->K);
  const int cb = d->C % 16 ? 4 : 16;
  if (cb == 4 && (d->KW > 8 || d->KH > 31))
    return fail(UNIT_E_ARG, "%s: 4-channel blocks need KW <= 8 and KH <= 31 (got %d x %d)", what, d->KH, d->KW);
  if (d->KD > d->D || d->KH > d->H || d->KW > d->W) return fail(UNIT_E_ARG, "%s: kernel window larger than the input", what);
  if (d->D >= 16384 || d->H >= 16384 || d->W >= 16384) return fail(UNIT_E_ARG, "%s: spatial extent too large", what);
  const int OD = (d->D - d->KD) / d->stride + 1, OH = (d->H - d->KH) / d->stride + 1, OW = (d->W - d->KW) / d->stride + 1;
  const int cc = d->C / cb;
  const size_t img = (size_t)cc * d->D * d->H * d->W * cb, opix = (size_t)OD * OH * OW, npix = opix * d->N;
  const size_t taps = (size_t)cc * d->KD * d->KH * d->KW;
  if (const size_t out_img = opix * d->K * 4, big = img > out_img ? img : out_img;
      d->N > 1 && big * d->N > kMaxTensorBytes && big <= kMaxTensorBytes) {
    // beyond the 32-bit offsets: one launch per slice of the batch (volumes lie one after the other)
    const int per = (int)(kMaxTensorBytes / big);
    unit_conv3d_desc sd = *d;
    for (int n0 = 0; n0 < d->N; n0 += per) {
      sd.N = d->N - n0 < per ? d->N - n0 : per;
      if (int rc = unit_conv3d_ncdhwc_s8s8s32(&sd, static_cast<const char *>(data) + (size_t)n0 * img, weight,
                                              static_cast<char *>(out) + (size_t)n0 * out_img, stream))
        return rc;
    }
    return UNIT_OK;
  }
  if (!fits(img * d->N) || npix > kMaxTensorBytes || !fits((size_t)d->K * taps * cb) || !fits(npix * d->K * 4))
    return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {data, weight, out})) return rc;
  if (int rc = check_device()) return rc;
  ConvGeom g;
  g.N = d->N; g.H = d->H; g.W = d->W; g.OH = OH; g.OW = OW;
  g.KH = d->KH; g.KW = d->KW; g.sh = g.sw = d->stride; g.pt = g.pl = 0; g.dh = g.dw = 1;
  g.npix = (int)npix;
  g.ntaps = (int)taps;
  g.ntab = g.ntaps;
  g.c4_steps = cc * d->KD * d->KH;
  g.img_bytes = (u32)img;
  g.by_ohw = FastDiv::make((int)opix);
  g.by_ow = FastDiv::make(OW);
  g.by_kh = FastDiv::make(d->KH);
  g.by_kw = FastDiv::make(d->KW);
  g.D = d->D; g.KD = d->KD; g.sd = d->stride; g.nopad = 1;
  g.by_plane = FastDiv::make(OH * OW);
  g.by_kd = FastDiv::make(d->KD);
  g.row_ones = 0;  // no padding: no window positions to mask
  // the launcher only reads K from the 2-D descriptor; the planner keys on pixels, channels and reduction length
  unit_conv_desc d2{d->N, d->C, d->H, d->W, d->K, d->KH, d->KW, d->stride, d->stride, 0, 0, 0, 0, 1, 1, cb};
  ConvPlan p = plan_conv(&d2, g.npix, g.ntaps * cb, nullptr, 0, true, true);
  if (!kConvTiles[p.variant].direct) p = heuristic_plan(g.npix, d->K, g.ntaps * cb, true, true, d->stride > 1);
  p.splits = 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (cb == 4) return conv_c4_direct(what, p, &d2, g, data, weight, nullptr, 1, false, out, s);
  return conv_s8_direct(what, p, &d2, g, data, weight, nullptr, 1, out, s);
}
