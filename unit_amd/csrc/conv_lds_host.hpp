// Host side of the LDS-shared convolution variants (conv_lds.hpp): launch and variant dispatch.
#pragma once
#include "conv_lds.hpp"
#include "conv_plan.hpp"
#include "conv_prepare.hpp"

namespace unit {

template <class S, bool SHIFT, bool Q8 = false, bool NCHW = false, class Op = OpI8>
int run_lds(const char *what, const char *tag, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
            const char *zero, const int *bias, int scale, void *out, const ConvPlan &plan, hipStream_t s,
            const int *bias2 = nullptr, int shift = 0, int planar = 0) {
  static_assert(S::kMain + 4096 <= kMaxLds, "variant does not fit the LDS");
  const PreparedLayout pl = prepared_layout(d->K, d->C, d->KH, d->KW, 16, Op::kInt ? 1 : 2);
  const int lds = S::kMain + S::RG * (d->KH * d->KW + 1) * 256;  // rings (or write-back areas) + position table
  if (lds > kMaxLds) return fail(UNIT_E_ARG, "%s: needs %d bytes of LDS (limit %d)", what, lds, kMaxLds);
  auto kern = conv_lds<S, SHIFT, Q8, NCHW, Op>;
  static thread_local bool allowed = false;  // the opt-in for > 64 KiB of dynamic LDS is sticky per kernel
  if (!allowed && lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
    allowed = true;
  }
  typename ConvEpilogue<Op>::Params ep{out, d->K, g.OH * g.OW, g.npix, g.by_ohw, bias, scale, bias2, shift, planar};
  const int gx = ceil_div(d->K, S::BX), gy = ceil_div(g.npix, S::BY);
  const int panel = plan.panel > 0 && plan.panel < gx ? plan.panel : 0;
  const GridMap gm = GridMap::make(gx, gy, panel ? panel : gx, 1);
  char tail[16] = "";
  if (panel) snprintf(tail, sizeof tail, "_r%d", panel);
  set_variant("%s_x%d_y%d_w%dx%d_g%d_k%d_r%d%s_s1", tag, S::BX, S::BY, S::WX, S::WY, S::KG, S::KS, S::NST, tail);
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(S::NT), lds, s, static_cast<const char *>(data),
                     static_cast<const char *>(w), zero, ep, g, gm, pl.nsteps);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  return UNIT_OK;
}

}  // namespace unit
