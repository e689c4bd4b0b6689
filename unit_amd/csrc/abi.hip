// C-ABI plumbing: version, thread-local error / variant strings, device check, convolution
// geometry validation, and the single-instruction MFMA diagnostics.
#include <stdlib.h>

#include "host.hpp"
#include "trace.hpp"
#include "loaders.hpp"

namespace unit {

char *error_buf() {
  static thread_local char buf[256] = "";
  return buf;
}

char *variant_buf() {
  static thread_local char buf[96] = "";
  return buf;
}

int tuning_override(const char *name) {
  const char *v = getenv(name);
  return v ? atoi(v) : 0;
}

int check_device() {
  static thread_local int cached_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(UNIT_E_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev == cached_dev) return UNIT_OK;
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return fail(UNIT_E_DEVICE, "hipGetDeviceProperties: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(UNIT_E_DEVICE, "device %d is %s; this library is built for gfx950 only", dev, prop.gcnArchName);
  cached_dev = dev;
  return UNIT_OK;
}

static int out_hw(const unit_conv_desc *d, int *OH, int *OW, const char *what) {
  if (d->N <= 0 || d->C <= 0 || d->H <= 0 || d->W <= 0 || d->K <= 0 || d->KH <= 0 || d->KW <= 0)
    return fail(UNIT_E_ARG, "%s: N, C, H, W, K, KH, KW must be positive", what);
  if (d->sh <= 0 || d->sw <= 0 || d->dh <= 0 || d->dw <= 0)
    return fail(UNIT_E_ARG, "%s: strides and dilations must be positive", what);
  if (d->pt < 0 || d->pl < 0 || d->pb < 0 || d->pr < 0) return fail(UNIT_E_ARG, "%s: negative padding", what);
  // the staged loaders mark a tap past the reduction end by a row offset of 32767, which must stay outside the
  // padded image for every output row
  if (d->pt >= 16384 || d->pl >= 16384 || d->pb >= 16384 || d->pr >= 16384)
    return fail(UNIT_E_ARG, "%s: padding of 16384 or more is not supported", what);
  const long eh = (long)d->H + d->pt + d->pb - (long)d->dh * (d->KH - 1) - 1;
  const long ew = (long)d->W + d->pl + d->pr - (long)d->dw * (d->KW - 1) - 1;
  if (eh < 0 || ew < 0) return fail(UNIT_E_ARG, "%s: kernel window larger than the padded input", what);
  *OH = (int)(eh / d->sh) + 1;
  *OW = (int)(ew / d->sw) + 1;
  return UNIT_OK;
}

// tapb: bytes one input pixel contributes per tap (u8 cb16: 16, u8 cb4: 4, f16 cb16: 32)
int conv_geom(const unit_conv_desc *d, int tapb, ConvGeom *g, const char *what) {
  int OH, OW;
  if (int rc = out_hw(d, &OH, &OW, what)) return rc;
  if (d->C % d->cb) return fail(UNIT_E_ARG, "%s: C (%d) must be a multiple of cb (%d)", what, d->C, d->cb);
  if (d->K % 16) return fail(UNIT_E_ARG, "%s: K (%d) must be a multiple of 16", what, d->K);
  if (d->H >= 16384 || d->W >= 16384 || (long)d->KH * d->dh >= 16384 || (long)d->KW * d->dw >= 16384)
    return fail(UNIT_E_ARG, "%s: spatial extent too large", what);
  const int cc = d->C / d->cb;
  const size_t img = (size_t)cc * d->H * d->W * tapb;
  const size_t npix = (size_t)d->N * OH * OW;
  if (!fits(img * d->N) || npix > kMaxTensorBytes || !fits((size_t)d->K * cc * d->KH * d->KW * tapb))
    return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  g->N = d->N;
  g->H = d->H;
  g->W = d->W;
  g->OH = OH;
  g->OW = OW;
  g->KH = d->KH;
  g->KW = d->KW;
  g->sh = d->sh;
  g->sw = d->sw;
  g->pt = d->pt;
  g->pl = d->pl;
  g->dh = d->dh;
  g->dw = d->dw;
  g->npix = (int)npix;
  g->ntaps = cc * d->KH * d->KW;
  g->ntab = g->ntaps;
  g->c4_steps = cc * d->KH;
  g->img_bytes = (u32)img;
  g->by_ohw = FastDiv::make(OH * OW);
  g->by_ow = FastDiv::make(OW);
  g->by_kh = FastDiv::make(d->KH);
  g->by_kw = FastDiv::make(d->KW);
  g->D = g->KD = g->sd = 1;
  g->nopad = !(d->pt || d->pl || d->pb || d->pr);
  g->by_plane = g->by_ohw;
  g->by_kd = FastDiv::make(1);
  g->row_ones = 0;
  if (d->dh == 1 && d->dw == 1 && d->KH * d->KW <= 31)
    for (int kh = 0; kh < d->KH; ++kh) g->row_ones |= 1u << (kh * d->KW);
  return UNIT_OK;
}

namespace {

// a (32, 32) s8 row-major, b (32, 32) s8 with row = output column; c (32, 32) i32 = a . b^T
__global__ __launch_bounds__(64) void mfma_tile_i8(const char *a, const char *b, int *c) {
  const int l = threadIdx.x, l32 = l & 31, half = l >> 5;
  v4i x = *reinterpret_cast<const v4i *>(a + l32 * 32 + half * 16);
  v4i y = *reinterpret_cast<const v4i *>(b + l32 * 32 + half * 16);
  v16i acc;
  for (int r = 0; r < 16; ++r) acc[r] = 0;
  acc = OpI8::mma(x, y, acc);
  for (int r = 0; r < 16; ++r) c[(8 * (r >> 2) + 4 * half + (r & 3)) * 32 + l32] = acc[r];
}

__global__ __launch_bounds__(64) void mfma_tile_f16(const char *a, const char *b, float *c) {
  const int l = threadIdx.x, l32 = l & 31, half = l >> 5;
  v4i x = *reinterpret_cast<const v4i *>(a + l32 * 32 + half * 16);
  v4i y = *reinterpret_cast<const v4i *>(b + l32 * 32 + half * 16);
  v16f acc;
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  acc = OpF16::mma(x, y, acc);
  for (int r = 0; r < 16; ++r) c[(8 * (r >> 2) + 4 * half + (r & 3)) * 32 + l32] = acc[r];
}

// Register-only MFMA throughput probe in the manner of poc/vnni/micro.cc:16-51: 4 independent
// accumulator chains per wave, no memory traffic; one workgroup of 4 waves per launch slot.
// RANDOM: four operand pairs of hashed bits, rotated so that consecutive MFMAs see different data
// GAUSS (fp16): the operands of the 4096^3 benchmark instead, x ~ N(0,1)/64 and y ~ N(0,1) (Box-Muller on the hashes)
template <class Op, bool RANDOM, bool GAUSS = false>
__global__ __launch_bounds__(256) void mfma_peak(int iters, typename Op::out_t *sink) {
  const int l = threadIdx.x;
  v4i xs[4], ys[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    xs[i] = v4i{l, l + 1, l + 2, l + 3};
    ys[i] = v4i{l ^ 5, l ^ 9, l ^ 3, l ^ 7};
    if (!Op::kInt) xs[i] = ys[i] = v4i{0x3c003c00, 0x3c003c00, 0x3c003c00, 0x3c003c00};
    if (RANDOM) {
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        u32 h = (u32)(l * 32 + i * 8 + d) * 2654435761u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13; h *= 3266489917u; h ^= h >> 16;
        u32 g = h * 2654435761u + 0x9e3779b9u;
        g ^= g >> 15; g *= 2246822519u; g ^= g >> 13;
        xs[i][d] = (int)(Op::kInt ? h : (h & 0x3fff3fffu));  // fp16: finite values below 2
        ys[i][d] = (int)(Op::kInt ? g : (g & 0x3fff3fffu));
        if constexpr (GAUSS) {
          auto pair = [](u32 u, float scale) {  // two normal values from one hash
            const float r = sqrtf(-2.f * __logf(((u & 0xffffu) + 1u) * (1.f / 65537.f))) * scale;
            const float t = (float)(u >> 16) * (6.2831853f / 65536.f);
            const _Float16 lo = (_Float16)(r * __cosf(t)), hi = (_Float16)(r * __sinf(t));
            return (int)((u32)__builtin_bit_cast(unsigned short, lo) | ((u32)__builtin_bit_cast(unsigned short, hi) << 16));
          };
          xs[i][d] = pair(h, 1.f / 64.f);
          ys[i][d] = pair(g, 1.f);
        }
      }
    }
  }
  typename Op::acc_t a0, a1, a2, a3;
  for (int r = 0; r < 16; ++r) a0[r] = a1[r] = a2[r] = a3[r] = 0;
  for (int i = 0; i < iters; ++i) {
    a0 = Op::mma(xs[0], ys[1], a0);
    a1 = Op::mma(xs[1], ys[2], a1);
    a2 = Op::mma(xs[2], ys[3], a2);
    a3 = Op::mma(xs[3], ys[0], a3);
  }
  typename Op::out_t s = 0;
  for (int r = 0; r < 16; ++r) s += a0[r] + a1[r] + a2[r] + a3[r];
  if (s == (typename Op::out_t)12345) sink[0] = s;  // keeps the chains alive; practically never taken
}

}  // namespace
}  // namespace unit

extern "C" int unit_mfma_peak(int32_t f16, int32_t blocks, int32_t iters, void *sink, unit_stream_t stream) {
  using namespace unit;
  if (!sink || blocks <= 0 || iters <= 0) return fail(UNIT_E_ARG, "unit_mfma_peak: bad arguments");
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if ((f16 & 7) == 5) {  // fp16 operands distributed like the 4096^3 benchmark's
    hipLaunchKernelGGL((mfma_peak<OpF16, true, true>), dim3(blocks), dim3(256), 0, s, iters, static_cast<float *>(sink));
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "unit_mfma_peak: %s", hipGetErrorString(e));
  }
  switch (f16 & 3) {
    case 0: hipLaunchKernelGGL((mfma_peak<OpI8, false>), dim3(blocks), dim3(256), 0, s, iters, static_cast<int *>(sink)); break;
    case 1: hipLaunchKernelGGL((mfma_peak<OpF16, false>), dim3(blocks), dim3(256), 0, s, iters, static_cast<float *>(sink)); break;
    case 2: hipLaunchKernelGGL((mfma_peak<OpI8, true>), dim3(blocks), dim3(256), 0, s, iters, static_cast<int *>(sink)); break;
    default: hipLaunchKernelGGL((mfma_peak<OpF16, true>), dim3(blocks), dim3(256), 0, s, iters, static_cast<float *>(sink)); break;
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "unit_mfma_peak: %s", hipGetErrorString(e));
}

#ifdef UNIT_TRACE_BUILD
// the timeline build only (make trace): the device buffer the instrumented kernels write their stamps to
namespace unit {
static unsigned long long *g_trace_buffer = nullptr;
unsigned long long *trace_buffer() { return g_trace_buffer; }
}  // namespace unit
extern "C" void unit_trace_set(void *device_buffer) { unit::g_trace_buffer = static_cast<unsigned long long *>(device_buffer); }
extern "C" int unit_trace_words(void) { return unit::kTraceWords; }
extern "C" int unit_trace_waves(void) { return unit::kTraceWaves; }
#endif

extern "C" int unit_version(void) { return 106; }  // 1.6: results stored sc1 nt, row-major int8 dense on the direct-to-LDS kernel, unit_mfma_peak mode 5 (the fp16 benchmark's operand distribution); 1.5: fp16 GEMM k-splits through a workspace or the library's static scratch; 1.4: LDS-shared convolution variants (16 KiB of zeros behind prepared int8 weights), dense on a prepared weight

extern "C" const char *unit_last_error(void) { return unit::error_buf(); }

extern "C" const char *unit_last_variant(void) { return unit::variant_buf(); }

extern "C" int unit_conv_out_hw(const unit_conv_desc *d, int32_t *OH, int32_t *OW) {
  if (!d || !OH || !OW) return unit::fail(UNIT_E_ARG, "unit_conv_out_hw: null pointer");
  return unit::out_hw(d, OH, OW, "unit_conv_out_hw");
}

extern "C" int unit_mfma_tile_i8(const void *a, const void *b, void *c, unit_stream_t stream) {
  using namespace unit;
  if (!a || !b || !c) return fail(UNIT_E_ARG, "unit_mfma_tile_i8: null pointer");
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(mfma_tile_i8, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     static_cast<const char *>(a), static_cast<const char *>(b), static_cast<int *>(c));
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "unit_mfma_tile_i8: %s", hipGetErrorString(e));
}

extern "C" int unit_mfma_tile_f16(const void *a, const void *b, void *c, unit_stream_t stream) {
  using namespace unit;
  if (!a || !b || !c) return fail(UNIT_E_ARG, "unit_mfma_tile_f16: null pointer");
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(mfma_tile_f16, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     static_cast<const char *>(a), static_cast<const char *>(b), static_cast<float *>(c));
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "unit_mfma_tile_f16: %s", hipGetErrorString(e));
}
