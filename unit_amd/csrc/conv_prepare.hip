// One-time weight preparation for the direct convolution kernels, and the C-ABI entry points of
// the convolutions that take prepared weights.  The reference's compiled graphs do the same kind
// of work on the constant weight, outside the convolution: the transpose / reshape chain into the
// blocked layout (apps/cpu/relay/result.log:8-13) and the per-channel weight sum of the u8 shift
// (result.log:15-16); here both are folded into one buffer shaped for the MFMA fragments.
#include "conv_plan.hpp"
#include "conv_prepare.hpp"
#include "mma_core.hpp"

namespace unit {

int conv_geom(const unit_conv_desc *d, int tapb, ConvGeom *g, const char *what);  // abi.hip
const TunedConv *tuned_conv_i8_prepared(int *n);                                  // below
int conv_u8_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                     const int *addend, void *out, hipStream_t s);  // conv_prepared_u8.hip
int conv_u8_prepared_lds(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                         const char *zero, const int *addend, void *out, hipStream_t s);  // conv_lds_u8.hip
int conv_s8_prepared_lds(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                         const char *zero, const int *bias, int scale, void *out, int planar, hipStream_t s);  // conv_lds_s8.hip
int conv_q8_prepared_lds(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                         const char *zero, const int *addend, const int *bias, int scale, int shift, void *out,
                         hipStream_t s);  // conv_lds_q8.hip
int conv_f16_prepared_lds(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *a, const void *w,
                          void *out, hipStream_t s);  // conv_lds_f16.hip
int conv_s8_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                     const int *bias, int scale, void *out, int planar, hipStream_t s);  // conv_prepared_s8.hip
int conv_c4_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                     const int *addend, int scale, bool shift, void *out, int planar, hipStream_t s);  // conv_prepared_c4.hip
int conv_q8_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *data, const void *w,
                     const int *addend, const int *bias, int scale, int shift, void *out, hipStream_t s);  // conv_prepared_q8.hip
int conv_f16_prepared(const ConvPlan &plan, const unit_conv_desc *d, const ConvGeom &g, const void *a, const void *w,
                      void *out, hipStream_t s);  // conv_prepared_f16.hip

namespace {

// one workgroup (64 lanes) per (32-channel block, k-step): gathers the 1 KiB of fragments
__global__ __launch_bounds__(64) void prepare_i8(const char *__restrict__ w, char *__restrict__ out, int K, int ntaps,
                                                 int nsteps) {
  const int blk = blockIdx.x, kb = blk / nsteps, s = blk - kb * nsteps;
  const int lane = threadIdx.x, ko = kb * 32 + (lane & 31), t = 2 * s + (lane >> 5);
  v4i v = {0, 0, 0, 0};
  if (ko < K && t < ntaps) {
    const char *src = w + ((size_t)(ko >> 4) * ntaps + t) * 256 + (ko & 15) * 4;
#pragma unroll
    for (int d = 0; d < 4; ++d) v[d] = *reinterpret_cast<const int *>(src + d * 64);
  }
  *reinterpret_cast<v4i *>(out + ((size_t)blk * 64 + lane) * 16) = v;
}

// 4-channel blocks (K/16, C/4, KH, KW, 1, 16, 4): one workgroup per (32-channel block, ci * KH + kh),
// a lane gathers 4 consecutive taps of the row (zeros for kw >= KW)
__global__ __launch_bounds__(64) void prepare_i8_c4(const char *__restrict__ w, char *__restrict__ out, int K, int KH,
                                                    int KW, int nsteps) {
  const int blk = blockIdx.x, kb = blk / nsteps, s = blk - kb * nsteps;
  const int lane = threadIdx.x, ko = kb * 32 + (lane & 31), half = lane >> 5;
  const int cc = nsteps / KH;
  v4i v = {0, 0, 0, 0};
  if (ko < K) {
    const char *row = w + ((size_t)(ko >> 4) * cc * KH + s) * KW * 64 + (ko & 15) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int kw = 4 * half + e;
      if (kw < KW) v[e] = *reinterpret_cast<const int *>(row + kw * 64);
    }
  }
  *reinterpret_cast<v4i *>(out + ((size_t)blk * 64 + lane) * 16) = v;
}

// one wave per output channel: 128 * sum of its weights (a tap of a 16-output-channel block is
// `dwords` dwords per channel, 64 bytes apart)
__global__ __launch_bounds__(64) void prepare_i8_addend(const char *__restrict__ w, int *__restrict__ addend, int K,
                                                        int ntaps, int dwords, int *__restrict__ zero_line) {
  const int ko = blockIdx.x, lane = threadIdx.x;
  if (ko < 32) {  // the grid has 32 x kblocks >= 32 workgroups: each clears 1/32 of the zero region
    constexpr int per = kZeroLine / 4 / 32;
    for (int i = lane; i < per; i += 64) zero_line[ko * per + i] = 0;
  }
  int sum = 0;
  if (ko < K) {
    const size_t tapb = (size_t)dwords * 64;
    const char *src = w + (size_t)(ko >> 4) * ntaps * tapb + (ko & 15) * 4;
    for (int t = lane; t < ntaps; t += 64)
      for (int d = 0; d < dwords; ++d)
        sum = __builtin_amdgcn_sdot4(*reinterpret_cast<const int *>(src + t * tapb + d * 64), 0x01010101, sum, false);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
  if (lane == 0) addend[ko] = sum << 7;
}

__global__ __launch_bounds__(64) void prepare_f16(const char *__restrict__ w, char *__restrict__ out, int K, int ntaps) {
  const int blk = blockIdx.x, kb = blk / ntaps, s = blk - kb * ntaps;
  const int lane = threadIdx.x, ko = kb * 32 + (lane & 31), half = lane >> 5;
  v8h h;
#pragma unroll
  for (int k = 0; k < 8; ++k) h[k] = (_Float16)0;
  if (ko < K) {
    const char *src = w + ((size_t)(ko >> 4) * ntaps + s) * 512 + (ko & 15) * 2 + half * 256;
#pragma unroll
    for (int k = 0; k < 8; ++k) h[k] = *reinterpret_cast<const _Float16 *>(src + k * 32);
  }
  *reinterpret_cast<v8h *>(out + ((size_t)blk * 64 + lane) * 16) = h;
}

int check_weight_shape(const char *what, int K, int C, int KH, int KW, int cb, int elem_bytes, PreparedLayout *pl) {
  if (elem_bytes != 1 && elem_bytes != 2) return fail(UNIT_E_ARG, "%s: elem_bytes must be 1 (int8) or 2 (fp16), got %d", what, elem_bytes);
  if (cb != 16 && !(cb == 4 && elem_bytes == 1))
    return fail(UNIT_E_ARG, "%s: cb must be 16, or 4 for int8 (got %d)", what, cb);
  if (K <= 0 || C <= 0 || KH <= 0 || KW <= 0) return fail(UNIT_E_ARG, "%s: K, C, KH, KW must be positive", what);
  if (K % 16 || C % cb) return fail(UNIT_E_ARG, "%s: K must be a multiple of 16 and C of cb (got %d, %d)", what, K, C);
  if (cb == 4 && KW > 8) return fail(UNIT_E_ARG, "%s: 4-channel blocks have a prepared form for KW <= 8 (got %d)", what, KW);
  if (!fits((size_t)K * C * KH * KW * elem_bytes)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  *pl = prepared_layout(K, C, KH, KW, cb, elem_bytes);
  if (!fits(pl->total_bytes)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  return UNIT_OK;
}

// measured on MI355X by `python -m unit_amd.tune --prepared` (key: N*OH*OW, K, C, KH, KW, stride)
const TunedConv kTunedI8Prepared[] = {
#include "tuned_conv_i8_prepared.inc"
    {0, 0, 0, 0, 0, 0, 0, 0, 0},
};
const TunedConv kTunedF16Prepared[] = {
#include "tuned_conv_f16_prepared.inc"
    {0, 0, 0, 0, 0, 0, 0, 0, 0},
};

// Prepared weights exist for the direct kernels only: a table entry or override that names a
// staged variant falls back to the heuristic's direct choice.
// lds_ok: the entry point also has the LDS-shared kernels (int8, 16-channel blocks).
ConvPlan plan_prepared(const unit_conv_desc *d, const ConvGeom &g, int kbytes, const TunedConv *table, int ntable,
                       bool int8, bool lds_ok = false) {
  // the LDS-shared kernels keep a window's positions as a 32-bit set: larger windows (possible for fp16, whose direct
  // kernels have no such limit) stay on the direct kernels, whatever a table row or an override names
  lds_ok = lds_ok && d->cb == 16 && d->KH * d->KW <= 31;
  ConvPlan p = plan_conv(d, g.npix, kbytes, table, ntable, int8, true, false, lds_ok);
  const TileShape &t = kConvTiles[p.variant];
  if (!(t.direct || (t.lds && lds_ok))) p = heuristic_plan(g.npix, d->K, kbytes, int8, true, d->sh * d->sw > 1);
  p.splits = 1;
  return p;
}

int check_prepared_conv(const char *what, const unit_conv_desc *d, int tapb, ConvGeom *g, const void *data,
                        const void *prepared, const void *out) {
  if (d->cb != 16 && !(d->cb == 4 && tapb == 16))
    return fail(UNIT_E_ARG, "%s: cb must be 16, or 4 for int8 (got %d)", what, d->cb);
  if (d->cb == 4) {
    if (d->KW > 8 || d->KH > 31 || d->dw != 1)
      return fail(UNIT_E_ARG, "%s: 4-channel blocks need KW <= 8, KH <= 31 and no dilation along W", what);
    tapb = 4;
  }
  if (int rc = conv_geom(d, tapb, g, what)) return rc;
  if (tapb == 16 && d->KH * d->KW > 31) return fail(UNIT_E_ARG, "%s: window of %d x %d exceeds 31 positions", what, d->KH, d->KW);
  if (!fits((size_t)g->npix * d->K * 4)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {data, prepared, out})) return rc;
  return check_device();
}

}  // namespace
}  // namespace unit

extern "C" int unit_conv2d_prepared_weight_bytes(int32_t K, int32_t C, int32_t KH, int32_t KW, int32_t cb,
                                                 int32_t elem_bytes, size_t *bytes) {
  using namespace unit;
  const char *what = "unit_conv2d_prepared_weight_bytes";
  if (!bytes) return fail(UNIT_E_ARG, "%s: null pointer", what);
  PreparedLayout pl;
  if (int rc = check_weight_shape(what, K, C, KH, KW, cb, elem_bytes, &pl)) return rc;
  *bytes = pl.total_bytes;
  return UNIT_OK;
}

extern "C" int unit_conv2d_prepare_weight(int32_t K, int32_t C, int32_t KH, int32_t KW, int32_t cb, int32_t elem_bytes,
                                          const void *weight, void *prepared, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv2d_prepare_weight";
  if (!weight || !prepared) return fail(UNIT_E_ARG, "%s: null pointer", what);
  PreparedLayout pl;
  if (int rc = check_weight_shape(what, K, C, KH, KW, cb, elem_bytes, &pl)) return rc;
  if (int rc = check_aligned(what, {weight, prepared})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int ntaps = (C / cb) * KH * KW;
  const char *w = static_cast<const char *>(weight);
  char *out = static_cast<char *>(prepared);
  if (elem_bytes == 1) {
    if (cb == 4)
      hipLaunchKernelGGL(prepare_i8_c4, dim3(pl.kblocks * pl.nsteps), dim3(64), 0, s, w, out, K, KH, KW, pl.nsteps);
    else
      hipLaunchKernelGGL(prepare_i8, dim3(pl.kblocks * pl.nsteps), dim3(64), 0, s, w, out, K, ntaps, pl.nsteps);
    hipLaunchKernelGGL(prepare_i8_addend, dim3(pl.kblocks * 32), dim3(64), 0, s, w,
                       reinterpret_cast<int *>(out + pl.frag_bytes), K, ntaps, cb / 4,
                       reinterpret_cast<int *>(out + pl.zero_off));
  } else {
    hipLaunchKernelGGL(prepare_f16, dim3(pl.kblocks * pl.nsteps), dim3(64), 0, s, w, out, K, ntaps);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  set_variant("prepare_%s_k%d_s%d", elem_bytes == 2 ? "f16" : (cb == 4 ? "i8c4" : "i8"), pl.kblocks, pl.nsteps);
  return UNIT_OK;
}

extern "C" int unit_conv2d_nchwc_u8s8s32_prepared(const unit_conv_desc *d, const void *data, const void *prepared,
                                                  void *out, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv2d_nchwc_u8s8s32_prepared";
  if (!d || !data || !prepared || !out) return fail(UNIT_E_ARG, "%s: null pointer", what);
  size_t in_img, out_img;
  if (const int per = batch_slice(d, (size_t)d->C, (size_t)d->K * 4, &in_img, &out_img))
    return run_batch_slices(d, per, in_img, out_img, data, out, [&](const unit_conv_desc *sd, const void *x, void *y) {
      return unit_conv2d_nchwc_u8s8s32_prepared(sd, x, prepared, y, stream);
    });
  ConvGeom g;
  if (int rc = check_prepared_conv(what, d, 16, &g, data, prepared, out)) return rc;
  const PreparedLayout pl = prepared_layout(d->K, d->C, d->KH, d->KW, d->cb, 1);
  const int ntable = (int)(sizeof(kTunedI8Prepared) / sizeof(kTunedI8Prepared[0])) - 1;
  const ConvPlan p = plan_prepared(d, g, g.ntaps * d->cb, kTunedI8Prepared, ntable, true, true);
  const char *w = static_cast<const char *>(prepared);
  const int *addend = reinterpret_cast<const int *>(w + pl.frag_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (d->cb == 4) return conv_c4_prepared(p, d, g, data, w, addend, 1, true, out, 0, s);
  if (kConvTiles[p.variant].lds) return conv_u8_prepared_lds(p, d, g, data, w, w + pl.zero_off, addend, out, s);
  return conv_u8_prepared(p, d, g, data, w, addend, out, s);
}

extern "C" int unit_conv2d_nchwc_u8s8u8_requant_prepared(const unit_conv_desc *d, const void *data, const void *prepared,
                                                         const int32_t *bias, int32_t scale, int32_t shift, void *out,
                                                         unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv2d_nchwc_u8s8u8_requant_prepared";
  if (!d || !data || !prepared || !out) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (shift < 1 || shift > 62) return fail(UNIT_E_ARG, "%s: shift must be in 1..62 (got %d)", what, shift);
  size_t in_img, out_img;
  if (const int per = batch_slice(d, (size_t)d->C, (size_t)d->K, &in_img, &out_img))
    return run_batch_slices(d, per, in_img, out_img, data, out, [&](const unit_conv_desc *sd, const void *x, void *y) {
      return unit_conv2d_nchwc_u8s8u8_requant_prepared(sd, x, prepared, bias, scale, shift, y, stream);
    });
  ConvGeom g;
  if (int rc = check_prepared_conv(what, d, 16, &g, data, prepared, out)) return rc;
  const PreparedLayout pl = prepared_layout(d->K, d->C, d->KH, d->KW, d->cb, 1);
  const int ntable = (int)(sizeof(kTunedI8Prepared) / sizeof(kTunedI8Prepared[0])) - 1;
  const ConvPlan p = plan_prepared(d, g, g.ntaps * d->cb, kTunedI8Prepared, ntable, true, true);
  const char *w = static_cast<const char *>(prepared);
  // (v * scale + 2^(shift-1)) >> shift is unchanged when scale doubles and shift grows by one; with
  // shift >= 33 the kernel needs only the high dword of the product
  while (shift < 33 && scale >= -(1 << 30) && scale < (1 << 30)) {
    scale *= 2;
    ++shift;
  }
  if (kConvTiles[p.variant].lds)
    return conv_q8_prepared_lds(p, d, g, data, w, w + pl.zero_off, reinterpret_cast<const int *>(w + pl.frag_bytes), bias,
                                scale, shift, out, static_cast<hipStream_t>(stream));
  return conv_q8_prepared(p, d, g, data, w, reinterpret_cast<const int *>(w + pl.frag_bytes), bias, scale, shift, out,
                          static_cast<hipStream_t>(stream));
}

namespace unit {
namespace {

// planar: 0 = blocked output, else the channel count of the (N, planar, OH, OW) output
int fused_prepared(const char *what, const unit_conv_desc *d, const void *data, const void *prepared,
                   const int32_t *bias, int32_t scale, void *out, int planar, unit_stream_t stream) {
  if (!d || !data || !prepared || !out) return fail(UNIT_E_ARG, "%s: null pointer", what);
  size_t in_img, out_img;
  if (const int per = batch_slice(d, (size_t)d->C, (size_t)d->K * 4, &in_img, &out_img)) {
    if (planar) out_img = out_img / d->K * planar;  // sliced as the blocked result would be; an image is planar channels
    return run_batch_slices(d, per, in_img, out_img, data, out, [&](const unit_conv_desc *sd, const void *x, void *y) {
      return fused_prepared(what, sd, x, prepared, bias, scale, y, planar, stream);
    });
  }
  ConvGeom g;
  if (int rc = check_prepared_conv(what, d, 16, &g, data, prepared, out)) return rc;
  const int ntable = (int)(sizeof(kTunedI8Prepared) / sizeof(kTunedI8Prepared[0])) - 1;
  const ConvPlan p = plan_prepared(d, g, g.ntaps * d->cb, kTunedI8Prepared, ntable, true, true);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (d->cb == 4) return conv_c4_prepared(p, d, g, data, prepared, bias, scale, false, out, planar, s);
  if (kConvTiles[p.variant].lds) {
    const PreparedLayout pl = prepared_layout(d->K, d->C, d->KH, d->KW, d->cb, 1);
    return conv_s8_prepared_lds(p, d, g, data, prepared, static_cast<const char *>(prepared) + pl.zero_off, bias, scale,
                                out, planar, s);
  }
  return conv_s8_prepared(p, d, g, data, prepared, bias, scale, out, planar, s);
}

}  // namespace
}  // namespace unit

extern "C" int unit_conv2d_nchwc_s8s8s32_fused_prepared(const unit_conv_desc *d, const void *data,
                                                        const void *prepared, const int32_t *bias, int32_t scale,
                                                        void *out, unit_stream_t stream) {
  return unit::fused_prepared("unit_conv2d_nchwc_s8s8s32_fused_prepared", d, data, prepared, bias, scale, out, 0, stream);
}

extern "C" int unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw(const unit_conv_desc *d, const void *data,
                                                             const void *prepared, const int32_t *bias, int32_t scale,
                                                             void *out, int32_t out_channels, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw";
  if (d && (out_channels <= d->K - 16 || out_channels > d->K))
    return fail(UNIT_E_ARG, "%s: out_channels %d does not round up to K = %d", what, out_channels, d->K);
  return fused_prepared(what, d, data, prepared, bias, scale, out, out_channels, stream);
}

extern "C" int unit_conv2d_nchw16c_f16f32_prepared(const unit_conv_desc *d, const void *a, const void *prepared,
                                                   void *out, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_conv2d_nchw16c_f16f32_prepared";
  if (!d || !a || !prepared || !out) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (d->pt || d->pl || d->pb || d->pr) return fail(UNIT_E_ARG, "%s: the operator has no padding argument; pre-pad the data", what);
  if (d->dh != 1 || d->dw != 1) return fail(UNIT_E_ARG, "%s: dilation must be 1", what);
  size_t in_img, out_img;
  if (const int per = batch_slice(d, (size_t)d->C * 2, (size_t)d->K * 4, &in_img, &out_img))
    return run_batch_slices(d, per, in_img, out_img, a, out, [&](const unit_conv_desc *sd, const void *x, void *y) {
      return unit_conv2d_nchw16c_f16f32_prepared(sd, x, prepared, y, stream);
    });
  ConvGeom g;
  if (int rc = check_prepared_conv(what, d, 32, &g, a, prepared, out)) return rc;
  const int ntable = (int)(sizeof(kTunedF16Prepared) / sizeof(kTunedF16Prepared[0])) - 1;
  const ConvPlan p = plan_prepared(d, g, g.ntaps * 32, kTunedF16Prepared, ntable, false, true);
  if (kConvTiles[p.variant].lds) return conv_f16_prepared_lds(p, d, g, a, prepared, out, static_cast<hipStream_t>(stream));
  return conv_f16_prepared(p, d, g, a, prepared, out, static_cast<hipStream_t>(stream));
}
