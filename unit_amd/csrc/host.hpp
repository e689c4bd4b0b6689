// Host-side helpers shared by the C-ABI translation units: error reporting, argument checks,
// kernel launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../../include/unit_amd.h"
#include "mma_core.hpp"

namespace unit {

char *error_buf();    // thread-local, 256 bytes
char *variant_buf();  // thread-local, 96 bytes

inline int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buf(), 256, fmt, ap);
  va_end(ap);
  return code;
}

inline void set_variant(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(variant_buf(), 96, fmt, ap);
  va_end(ap);
}

// Integer value of a tuning environment variable (0 when unset): lets a caller pin a kernel
// variant per process, as the reference pins schedule indices through tensorizer.tune globals
// (python/tensorizer/tune.py:3-16).
int tuning_override(const char *name);

int check_device();  // UNIT_OK or UNIT_E_DEVICE (message set)

constexpr size_t kMaxTensorBytes = 0x7fffffffull;
constexpr int kMaxLds = 160 * 1024;

inline bool fits(size_t bytes) { return bytes <= kMaxTensorBytes; }

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

template <class Op, class T, class XL, class YL, class Epi, int WS>
int launch_mma(const typename XL::Params &xp, const typename YL::Params &yp, const typename Epi::Params &ep,
               int nk, int gx, int gy, int ph, int aux_bytes, hipStream_t stream, const char *what) {
  const int lds = T::LDS_TILES + aux_bytes;
  if (lds > kMaxLds) return fail(UNIT_E_ARG, "%s: needs %d bytes of LDS (limit %d)", what, lds, kMaxLds);
  auto kern = mma_kernel<Op, T, XL, YL, Epi, WS>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
  GridMap gm;
  gm.gx = gx;
  gm.gy = gy;
  gm.ph = ph < 1 ? 1 : (ph > gx ? gx : ph);
  gm.total = gx * gy;
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(T::NT), lds, stream, xp, yp, ep, nk, gm);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  return UNIT_OK;
}

}  // namespace unit
