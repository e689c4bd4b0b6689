// Host side of the direct (no operand staging) convolution variants: launch and variant dispatch.
#pragma once
#include "conv_direct.hpp"
#include "conv_plan.hpp"

namespace unit {

template <class Op, class S, bool SHIFT, bool PREP = false, bool C4 = false, bool Q8 = false, bool NCHW = false>
int run_direct(const char *what, const char *tag, const unit_conv_desc *d, const ConvGeom &g, const void *data,
               const void *w, const int *bias, int scale, void *out, const ConvPlan &plan, hipStream_t s,
               const int *bias2 = nullptr, int shift = 0, int planar = 0) {
  const int ntab = C4 ? 2 * g.c4_steps : (Op::kInt ? 2 * ((g.ntaps + 1) / 2) : g.ntaps);
  const int lds = S::template lds_fixed<Op>() + ntab * 8;
  if (lds > kMaxLds) return fail(UNIT_E_ARG, "%s: needs %d bytes of LDS (limit %d)", what, lds, kMaxLds);
  auto kern = conv_direct<Op, S, SHIFT, PREP, C4, Q8, NCHW>;
  static thread_local int lds_allowed = 0;  // the opt-in for > 64 KiB of dynamic LDS is sticky per kernel
  if (lds > lds_allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
    lds_allowed = kMaxLds;
  }
  typename ConvEpilogue<Op>::Params ep{out, d->K, g.by_ohw.d, g.npix, g.by_ohw, bias, scale, bias2, shift, planar};
  const int gx = ceil_div(d->K, S::BX), gy = ceil_div(g.npix, S::BY);
  const int panel = plan.panel > 0 && plan.panel < gx ? plan.panel : 0;
  const GridMap gm = GridMap::make(gx, gy, panel ? panel : gx, 1);
  char tail[16] = "";
  if (panel) snprintf(tail, sizeof tail, "_r%d", panel);
  set_variant("%s_x%d_y%d_g%d_d%d%s%s%s_s1", tag, S::BX, S::BY, S::KG, S::D,
              S::kFourWaves ? "w4" : "", S::PAD ? "" : "n", tail);
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(S::NT), lds, s, static_cast<const char *>(data),
                     static_cast<const char *>(w), ep, g, gm UNIT_TRACE(, trace_buffer()));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  return UNIT_OK;
}

}  // namespace unit
