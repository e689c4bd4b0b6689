// Host-side helpers shared by the C-ABI translation units: error reporting, argument checks,
// kernel launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <initializer_list>

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

// The kernels move operands and results with 16-byte vector accesses: every tensor pointer handed
// to a compute entry point must be 16-byte aligned (framework allocators give 256 bytes or more).
inline int check_aligned(const char *what, std::initializer_list<const void *> ptrs) {
  for (const void *p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) % 16)
      return fail(UNIT_E_ARG, "%s: tensor pointers must be 16-byte aligned (got %p)", what, p);
  return UNIT_OK;
}

// Images per launch for a convolution whose data or result would pass the kernels' 32-bit offsets (0: the whole
// batch fits one launch, or a single image is already too large and the entry point's own checks reject it).
// Images lie one after the other in the blocked and in the planar layouts alike, so such a convolution runs as
// several launches over slices of the batch.  in_px / out_px: bytes per input / output pixel over all channels.
inline int batch_slice(const unit_conv_desc *d, size_t in_px, size_t out_px, size_t *in_img, size_t *out_img) {
  int32_t OH = 0, OW = 0;
  if (d->N <= 1 || unit_conv_out_hw(d, &OH, &OW) != UNIT_OK) return 0;
  *in_img = (size_t)d->H * d->W * in_px;
  *out_img = (size_t)OH * OW * out_px;
  const size_t big = *in_img > *out_img ? *in_img : *out_img;
  if (big * d->N <= kMaxTensorBytes || big > kMaxTensorBytes) return 0;
  return (int)(kMaxTensorBytes / big);
}

// call(desc, data, out) for each slice of `per` images; stops at the first error
template <class F>
int run_batch_slices(const unit_conv_desc *d, int per, size_t in_img, size_t out_img, const void *data, void *out,
                     F call) {
  unit_conv_desc s = *d;
  for (int n0 = 0; n0 < d->N; n0 += per) {
    s.N = d->N - n0 < per ? d->N - n0 : per;
    if (int rc = call(&s, static_cast<const char *>(data) + (size_t)n0 * in_img,
                      static_cast<char *>(out) + (size_t)n0 * out_img))
      return rc;
  }
  return UNIT_OK;
}

// Rows per launch for a GEMM whose row-major a (M, K) or c (M, N) would pass the 32-bit offsets (0: one launch, or a
// slice of 256 rows is already too large and the entry point rejects the call).  A multiple of 256, the tile height.
inline int row_slice(int M, size_t a_row_bytes, size_t c_row_bytes) {
  const size_t big = a_row_bytes > c_row_bytes ? a_row_bytes : c_row_bytes;
  if (big * M <= kMaxTensorBytes) return 0;
  const size_t rows = kMaxTensorBytes / big / 256 * 256;
  return rows < (size_t)M ? (int)rows : 0;
}

// call(a, c, rows) for each slice of `per` rows; stops at the first error
template <class F>
int run_row_slices(int M, int per, size_t a_row_bytes, size_t c_row_bytes, const void *a, void *c, F call) {
  for (int m0 = 0; m0 < M; m0 += per)
    if (int rc = call(static_cast<const char *>(a) + (size_t)m0 * a_row_bytes,
                      static_cast<char *>(c) + (size_t)m0 * c_row_bytes, M - m0 < per ? M - m0 : per))
      return rc;
  return UNIT_OK;
}

// k-splits of a GEMM.  Few output tiles and a long reduction leave most of the chip idle (the reference's own
// GEMM sizes, 128 x 768 x 3072 in apps/gpu/gemm.py:6 and 128 x 3072 x 768 in apps/cpu/kernel/int8-gemm.py:9, are 6
// and 24 tiles of 128 x 128; the reference splits the reduction of the first with rfactor, gemm.py:22-40): the
// reduction is then shared between workgroups that add their partial tiles with atomics into the zero-filled
// output.  Below 128 tiles of 128 x 128: about 128 workgroups in all, at least 256 reduction bytes each; up to
// 256 tiles, three splits when each still gets 2 KiB of reduction (measured: 256 x 8192 x 8192 fp16 133 -> 67 us).
// More tiles fill the chip by themselves, and the atomics (output bytes x splits) then cost more than they gain.
// Exact for int32; for fp32 the order of the additions varies from run to run (last-bit differences).
// The environment variable pins the count (1 = off).  kbytes: reduction bytes per row; nk: stages of the tile.
inline int gemm_k_splits(const char *env, int M, int N, long kbytes, int nk) {
  int splits = tuning_override(env);
  if (splits <= 0) {
    const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
    splits = 1;
    if (tiles < 128)
      splits = (int)(128 / tiles < kbytes / 256 ? 128 / tiles : kbytes / 256);
    else if (tiles < 256 && kbytes >= 6144)
      splits = 3;
  }
  return splits < 1 ? 1 : (splits > nk ? nk : splits);
}

// Which all-direct GEMM tile (both operands global -> LDS): 256 x 256 (eight waves, one workgroup per CU, the least LDS
// traffic per MFMA) or 128 x 128 (four waves, two workgroups per CU).  Measured time per 2048 reduction bytes (fp16):
// a round of large tiles 30 us (24 when under 200 CUs are busy), a round of 512 small tiles 21.5 us, 13 us when at
// most 256 are left (one per CU).
inline bool direct_gemm_large_tiles(int M, int N) {
  const long tb = (long)ceil_div(M, 256) * ceil_div(N, 256), t128 = (long)ceil_div(M, 128) * ceil_div(N, 128);
  const double big = (double)((tb + 255) / 256) * (tb <= 200 ? 24.0 : 30.0);
  const long rest = t128 % 512;
  const double small = (double)(t128 / 512) * 21.5 + (rest == 0 ? 0.0 : rest <= 256 ? 13.0 : 21.5);
  return M >= 256 && N >= 256 && big < small;
}

// k-splits of the 128 x 128 all-direct tiles (results added with atomics into the zero-filled output): up to 128
// workgroups, and a split's share of the reduction at least 32 bytes x the tile count (the zero fill and the atomics
// cost in proportion to the output: fp16 1024^3 on 64 tiles runs 14.5 us whole and 15.6 us in two splits,
// 512 x 512 x 4096 on 16 tiles 35 us whole and 15 us in 8).  The environment variable pins the count.
inline int direct_gemm_k_splits(const char *env, int M, int N, long kbytes) {
  int splits = tuning_override(env);
  if (splits <= 0) {
    const long t128 = (long)ceil_div(M, 128) * ceil_div(N, 128);
    const long share = 32 * t128 > 256 ? 32 * t128 : 256;
    splits = (int)(128 / t128 < kbytes / share ? 128 / t128 : kbytes / share);
  }
  return splits < 1 ? 1 : splits;
}

// Enqueue mma_kernel over gx x gy tiles and `splits` k-ranges.  With splits > 1 the epilogue
// accumulates with atomics, so `out` (out_bytes, a multiple of 16) is zero-filled first.
template <class Op, class T, class XL, class YL, class Epi, int WS>
int launch_mma(const typename XL::Params &xp, const typename YL::Params &yp, const typename Epi::Params &ep,
               int nk, int gx, int gy, int ph, int splits, void *out, size_t out_bytes, int aux_bytes,
               hipStream_t stream, const char *what) {
  constexpr int epi = Epi::template lds_bytes<T>() + T::XCHG;  // epilogue scratch + k-group hand-over
  const int lds = (T::LDS_TILES + aux_bytes) > epi ? (T::LDS_TILES + aux_bytes) : epi;
  if (lds > kMaxLds) return fail(UNIT_E_ARG, "%s: needs %d bytes of LDS (limit %d)", what, lds, kMaxLds);
  auto kern = mma_kernel<Op, T, XL, YL, Epi, WS>;
  // the opt-in for > 64 KiB of dynamic LDS is sticky per kernel; raise it only when needed
  static thread_local int lds_allowed = 0;
  if (lds > lds_allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
    lds_allowed = kMaxLds;
  }
  if (splits < 1) splits = 1;
  if (splits > nk) splits = nk;
  if (splits > 1 && !Epi::kSplitPlanes) {
    const size_t n16 = out_bytes / 16;
    hipLaunchKernelGGL(zero_fill, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, stream,
                       static_cast<v4i *>(out), n16);
  }
  const GridMap gm = GridMap::make(gx, gy, ph, splits);
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(T::NT), lds, stream, xp, yp, ep, nk, gm);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  return UNIT_OK;
}

}  // namespace unit
