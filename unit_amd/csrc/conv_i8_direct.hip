// Host side of the direct (no operand staging) int8 NCHW16c convolution variants.
#include "conv_direct.hpp"
#include "conv_plan.hpp"

namespace unit {
namespace {

template <class S>
int run_direct(const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w, void *out,
               const ConvPlan &plan, hipStream_t s) {
  const char *what = "unit_conv2d_nchwc_u8s8s32";
  const int nsteps = (g.ntaps + 1) / 2;
  const int lds = S::LDS_FIXED + 2 * nsteps * 8;
  if (lds > kMaxLds) return fail(UNIT_E_ARG, "%s: needs %d bytes of LDS (limit %d)", what, lds, kMaxLds);
  auto kern = conv_direct_i8<S>;
  static thread_local int lds_allowed = 0;  // the opt-in for > 64 KiB of dynamic LDS is sticky per kernel
  if (lds > lds_allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
    lds_allowed = kMaxLds;
  }
  ConvEpilogue<OpI8>::Params ep{out, d->K, g.OH * g.OW, g.npix, g.by_ohw};
  GridMap gm;
  gm.gx = ceil_div(d->K, S::BX);
  gm.gy = ceil_div(g.npix, S::BY);
  const int panel = plan.panel > 0 && plan.panel < gm.gx ? plan.panel : 0;
  gm.ph = panel ? panel : gm.gx;
  gm.splits = 1;
  gm.total = gm.gx * gm.gy;
  char tail[16] = "";
  if (panel) snprintf(tail, sizeof tail, "_r%d", panel);
  set_variant("i8direct_c16_x%d_y%d_g%d_d%d%s%s_s1", S::BX, S::BY, S::KG, S::D, S::PAD ? "" : "n", tail);
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(S::NT), lds, s, static_cast<const char *>(data),
                     static_cast<const char *>(w), ep, g, gm);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  return UNIT_OK;
}

}  // namespace

int conv_i8_direct(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                   void *out, hipStream_t s) {
  if (d->cb != 16 || d->KH * d->KW > 31)
    return fail(UNIT_E_ARG, "unit_conv2d_nchwc_u8s8s32: kernel variant %d not available for this layout or window",
                plan.variant);
  // Without zero padding every tap of a valid pixel lies inside the image and the kernel without
  // tap masks serves; an odd tap count needs the masks too, for the tap that pads the last k-step.
  const bool masked = d->pt || d->pl || d->pb || d->pr || (g.ntaps & 1);
#define UNIT_CONV_VARIANT(ID, BX, BY, BKB, WX, WY, PF, FF, KG)
#define UNIT_CONV_DIRECT(ID, TX, TY, KG, D) \
  case ID:                                  \
    return masked ? run_direct<DirectShape<TX, TY, KG, D, true>>(d, g, data, w, out, plan, s) \
                  : run_direct<DirectShape<TX, TY, KG, D, false>>(d, g, data, w, out, plan, s);
  switch (plan.variant) {
#include "conv_variants.def"
    default:
      return fail(UNIT_E_ARG, "unit_conv2d_nchwc_u8s8s32: unknown kernel variant %d", plan.variant);
  }
#undef UNIT_CONV_DIRECT
#undef UNIT_CONV_VARIANT
}

}  // namespace unit
