// Layout transforms and weight pre-packs.  All are pure byte permutations bound by HBM traffic
// (read once + write once); none touches the MFMA unit.
#include "host.hpp"

namespace unit {
namespace {

// ---- NCHW <-> NCHW{CB}c -------------------------------------------------------------------
// A thread moves PP = 4 / ES consecutive pixels of one channel block: CB 4-byte words (one per
// channel plane, coalesced across lanes) <-> PP contiguous rows of CB elements.
template <int ES, int CB, bool PACK>
__global__ __launch_bounds__(256) void nchwc_words(const char *src, char *dst, int C, int HW, int cc,
                                                   int groups /* HW / PP */) {
  constexpr int PP = 4 / ES, ROWW = CB * ES / 4;  // words per output row
  const int g = blockIdx.x * 256 + threadIdx.x;
  if (g >= groups) return;
  const int plane = blockIdx.y;  // n * cc + ci
  const int n = plane / cc, ci = plane - n * cc;
  const size_t p0 = (size_t)g * PP;
  const char *nchw = PACK ? src : dst;
  u32 w[CB];
  u32 rows[PP][ROWW];
  if (PACK) {
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      const int ch = ci * CB + c;
      w[c] = ch < C ? *reinterpret_cast<const u32 *>(nchw + (((size_t)n * C + ch) * HW + p0) * ES) : 0u;
    }
#pragma unroll
    for (int pp = 0; pp < PP; ++pp)
#pragma unroll
      for (int j = 0; j < ROWW; ++j) {
        u32 v = 0;
#pragma unroll
        for (int e = 0; e < 4 / ES; ++e) {
          const u32 el = ES == 4 ? w[j] : (w[j * (4 / ES) + e] >> (8 * ES * pp)) & (ES == 1 ? 0xffu : 0xffffu);
          v |= el << (8 * ES * e);
        }
        rows[pp][j] = v;
      }
    char *o = dst + ((size_t)plane * HW + p0) * CB * ES;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp)
#pragma unroll
      for (int j = 0; j < ROWW; ++j) reinterpret_cast<u32 *>(o)[pp * ROWW + j] = rows[pp][j];
  } else {
    const char *in = src + ((size_t)plane * HW + p0) * CB * ES;
#pragma unroll
    for (int pp = 0; pp < PP; ++pp)
#pragma unroll
      for (int j = 0; j < ROWW; ++j) rows[pp][j] = reinterpret_cast<const u32 *>(in)[pp * ROWW + j];
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      u32 v = 0;
#pragma unroll
      for (int pp = 0; pp < PP; ++pp) {
        const u32 word = rows[pp][c * ES / 4];
        const u32 el = ES == 4 ? word : (word >> (8 * ES * (c % (4 / ES)))) & (ES == 1 ? 0xffu : 0xffffu);
        v |= el << (8 * ES * pp);
      }
      const int ch = ci * CB + c;
      if (ch < C) *reinterpret_cast<u32 *>(dst + (((size_t)n * C + ch) * HW + p0) * ES) = v;
    }
  }
}

// u8 / s8 with 16-channel blocks: a thread moves 16 pixels x 16 channels of one (image, channel block)
// plane, 16-byte loads and stores on both sides (16 consecutive pixels of one channel plane <-> one
// pixel's 16 channels) and a 16 x 16 byte transpose in registers: sixteen 4 x 4 transposes of
// two v_perm_b32 stages each.  Packing then passes the rows through a wave-private LDS area so that
// a store instruction writes 64 consecutive pixels (1 KiB) instead of 16-byte pieces 256 bytes
// apart; LDS operations of one wave execute in order, so the area needs no barrier.
// The work items are the 16-pixel groups of all planes in one flat index (small planes still fill
// the blocks); a plane of fewer than 16 pixels is one partial group that goes byte by byte on the
// NCHW side.
// 4 x 4 byte transpose: rows a, b, c, d (byte k of a row = column k) -> t[k] = {a.k, b.k, c.k, d.k}
__device__ __forceinline__ void transpose4x4(u32 a, u32 b, u32 c, u32 d, u32 (&t)[4]) {
  const u32 x0 = __builtin_amdgcn_perm(b, a, 0x05010400u), x1 = __builtin_amdgcn_perm(b, a, 0x07030602u);
  const u32 y0 = __builtin_amdgcn_perm(d, c, 0x05010400u), y1 = __builtin_amdgcn_perm(d, c, 0x07030602u);
  t[0] = __builtin_amdgcn_perm(y0, x0, 0x05040100u);
  t[1] = __builtin_amdgcn_perm(y0, x0, 0x07060302u);
  t[2] = __builtin_amdgcn_perm(y1, x1, 0x05040100u);
  t[3] = __builtin_amdgcn_perm(y1, x1, 0x07060302u);
}

// 16 bytes at any byte address (a group's first byte in a plane of H * W bytes)
typedef int bytes16_t __attribute__((ext_vector_type(4), aligned(1)));

template <bool PACK>
__global__ __launch_bounds__(256) void nchw16c_bytes(const char *src, char *dst, int C, int HW, int cc,
                                                     FastDiv by_groups /* ceil(HW / 16) */, int total_groups) {
  const int gid = blockIdx.x * 256 + threadIdx.x;
  if (!PACK && gid >= total_groups) return;
  const bool live = gid < total_groups;  // packing: lanes past the end still take part in the wave's write-back
  int plane, g;                          // plane = n * cc + ci
  by_groups.divmod(live ? gid : 0, plane, g);
  const int n = plane / cc, ci = plane - n * cc;
  // the last group of a plane is moved back to end with the plane (it overlaps its neighbour, and both
  // write the same bytes there); only planes of fewer than 16 pixels have a partial group
  const int p0 = g * 16 + 16 <= HW || HW < 16 ? g * 16 : HW - 16;
  const int cnt = live ? min(16, HW - p0) : 0;  // pixels of this group
  const char *nchw = PACK ? src : dst;
  const size_t chan0 = ((size_t)n * C + ci * 16) * HW + p0;  // byte offset of channel ci * 16, pixel p0
  const size_t flat0 = (size_t)plane * HW + p0;              // pixel index in the blocked tensor
  v4i planes[16];  // [channel]: 16 pixels
  v4i rows[16];    // [pixel]: 16 channels
  if (PACK) {
    if (cnt == 16) {
#pragma unroll
      for (int c = 0; c < 16; ++c)
        planes[c] = ci * 16 + c < C ? (v4i) * reinterpret_cast<const bytes16_t *>(nchw + chan0 + (size_t)c * HW) : v4i{0, 0, 0, 0};
    } else {
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        u32 w[4] = {0, 0, 0, 0};
        if (ci * 16 + c < C)
          for (int e = 0; e < cnt; ++e) w[e >> 2] |= (u32)(unsigned char)nchw[chan0 + (size_t)c * HW + e] << (8 * (e & 3));
        planes[c] = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32 t[4];
        transpose4x4(planes[4 * j][q], planes[4 * j + 1][q], planes[4 * j + 2][q], planes[4 * j + 3][q], t);
#pragma unroll
        for (int k = 0; k < 4; ++k) rows[4 * q + k][j] = (int)t[k];
      }
    // lane l parks its 16 rows at pitch 272 bytes (conflict-free both ways) with the group's first pixel and
    // pixel count behind them; the wave then stores row after row, 64 rows per instruction
    __shared__ __attribute__((aligned(16))) char stage[4][64 * 272];
    const int lane = threadIdx.x & 63;
    char *st = stage[threadIdx.x >> 6];
#pragma unroll
    for (int r = 0; r < 16; ++r) *reinterpret_cast<v4i *>(st + lane * 272 + r * 16) = rows[r];
    *reinterpret_cast<v2i *>(st + lane * 272 + 256) = v2i{(int)flat0, cnt};
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int pix = k * 64 + lane;
      const char *slot = st + (pix >> 4) * 272;
      const v4i v = *reinterpret_cast<const v4i *>(slot + (pix & 15) * 16);
      const v2i where = *reinterpret_cast<const v2i *>(slot + 256);
      if ((pix & 15) < where[1]) reinterpret_cast<v4i *>(dst)[(size_t)where[0] + (pix & 15)] = v;
    }
  } else {
    const v4i *blocked = reinterpret_cast<const v4i *>(src) + flat0;
#pragma unroll
    for (int r = 0; r < 16; ++r) rows[r] = r < cnt ? blocked[r] : v4i{0, 0, 0, 0};
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32 t[4];
        transpose4x4(rows[4 * q][j], rows[4 * q + 1][j], rows[4 * q + 2][j], rows[4 * q + 3][j], t);
#pragma unroll
        for (int k = 0; k < 4; ++k) planes[4 * j + k][q] = (int)t[k];
      }
    if (cnt == 16) {
#pragma unroll
      for (int c = 0; c < 16; ++c)
        if (ci * 16 + c < C) *reinterpret_cast<bytes16_t *>(dst + chan0 + (size_t)c * HW) = (bytes16_t)planes[c];
    } else {
#pragma unroll
      for (int c = 0; c < 16; ++c)
        if (ci * 16 + c < C)
          for (int e = 0; e < cnt; ++e) dst[chan0 + (size_t)c * HW + e] = (char)((u32)planes[c][e >> 2] >> (8 * (e & 3)));
    }
  }
}

// any shape / element size: one thread per blocked element
template <bool PACK>
__global__ __launch_bounds__(256) void nchwc_elems(const char *src, char *dst, int C, int HW, int cc, int cb,
                                                   int es, size_t total) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % cb);
  const size_t r = i / cb;
  const size_t p = r % HW, plane = r / HW;
  const int ci = (int)(plane % cc);
  const size_t n = plane / cc;
  const int ch = ci * cb + c;
  const size_t flat = ((n * C + ch) * HW + p) * es;
  for (int b = 0; b < es; ++b) {
    if (PACK)
      dst[i * es + b] = ch < C ? src[flat + b] : 0;
    else if (ch < C)
      dst[flat + b] = src[i * es + b];
  }
}

template <bool PACK>
int nchwc(const void *src, void *dst, int N, int C, int H, int W, int cb, int es, hipStream_t s, const char *what) {
  if (!src || !dst) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (N <= 0 || C <= 0 || H <= 0 || W <= 0) return fail(UNIT_E_ARG, "%s: N, C, H, W must be positive", what);
  if (cb <= 0 || cb > 64) return fail(UNIT_E_ARG, "%s: cb must be in 1..64 (got %d)", what, cb);
  if (es != 1 && es != 2 && es != 4) return fail(UNIT_E_ARG, "%s: elem_size must be 1, 2 or 4 (got %d)", what, es);
  const int cc = ceil_div(C, cb);
  const size_t hw = (size_t)H * W, total = (size_t)N * cc * hw * cb;
  if (const size_t img = (size_t)cc * hw * cb * es; N > 1 && !fits(total * es) && fits(img)) {
    // images lie one after the other on both sides: slices of the batch that fit 32-bit offsets
    const int per = (int)(kMaxTensorBytes / img);
    const size_t planar = (size_t)C * hw * es, src_img = PACK ? planar : img, dst_img = PACK ? img : planar;
    for (int n0 = 0; n0 < N; n0 += per)
      if (int rc = nchwc<PACK>(static_cast<const char *>(src) + n0 * src_img, static_cast<char *>(dst) + n0 * dst_img,
                               N - n0 < per ? N - n0 : per, C, H, W, cb, es, s, what))
        return rc;
    return UNIT_OK;
  }
  if (!fits(total * es)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_device()) return rc;
  const char *in = static_cast<const char *>(src);
  char *out = static_cast<char *>(dst);
  const int HW = (int)hw, pp = 4 / es;
  const bool words = HW % pp == 0 && (cb == 16 || (cb == 4 && es == 1)) && (size_t)N * cc <= 65535;
  if (es == 1 && cb == 16) {
    const int groups = ceil_div(HW, 16), total_groups = N * cc * groups;  // < 2^27: the tensor fits 2^31 bytes
    const dim3 grid(ceil_div(total_groups, 256));
    const FastDiv by_groups = FastDiv::make(groups);
    hipLaunchKernelGGL(nchw16c_bytes<PACK>, grid, dim3(256), 0, s, in, out, C, HW, cc, by_groups, total_groups);
  } else if (words) {
    const int groups = HW / pp;
    dim3 grid(ceil_div(groups, 256), N * cc);
#define UNIT_NCHWC(ES, CB)                                                                                   \
  hipLaunchKernelGGL((nchwc_words<ES, CB, PACK>), grid, dim3(256), 0, s, in, out, C, HW, cc, groups)
    if (es == 1 && cb == 16) UNIT_NCHWC(1, 16);
    else if (es == 1 && cb == 4) UNIT_NCHWC(1, 4);
    else if (es == 2) UNIT_NCHWC(2, 16);
    else UNIT_NCHWC(4, 16);
#undef UNIT_NCHWC
  } else {
    hipLaunchKernelGGL(nchwc_elems<PACK>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, in, out, C, HW,
                       cc, cb, es, total);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

// ---- weight pre-packs ---------------------------------------------------------------------
// dst[ko][ci][kh][kw][e][kb][i] = src[16ko+kb][cb*ci+4e+i][kh][kw]; one thread per dst dword
__global__ __launch_bounds__(256) void prepack_conv_s8(const signed char *src, int *dst, int O, int I, int KH,
                                                       int KW, int cb, int cc, size_t words) {
  const size_t wi = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (wi >= words) return;
  const int E = cb / 4;
  size_t r = wi;
  const int kb = (int)(r % 16);
  r /= 16;
  const int e = (int)(r % E);
  r /= E;
  const int kw = (int)(r % KW);
  r /= KW;
  const int kh = (int)(r % KH);
  r /= KH;
  const int ci = (int)(r % cc);
  const int ko = (int)(r / cc);
  const int o = 16 * ko + kb;
  u32 v = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int ic = cb * ci + 4 * e + i;
    if (o < O && ic < I) v |= (u32)(unsigned char)src[(((size_t)o * I + ic) * KH + kh) * KW + kw] << (8 * i);
  }
  dst[wi] = (int)v;
}

// dst[n/128][k/4][n%128][k%4] = src[n][k]; one thread per dword; a 128-thread row of the block
// reads 128 different rows n at the same k/4: 4-byte reads with stride K (served by L2), and
// writes 512 contiguous bytes
__global__ __launch_bounds__(256) void prepack_dense_s8(const int *src, int *dst, int K4, size_t words) {
  const size_t wi = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (wi >= words) return;
  const int nl = (int)(wi % 128);
  const size_t r = wi / 128;
  const int kg = (int)(r % K4);
  const size_t nb = r / K4;
  dst[wi] = src[(nb * 128 + nl) * K4 + kg];
}

// dst[oc][ic][x][y][ib][ob] = src[16oc+ob][16ic+ib][x][y]; one thread per element
__global__ __launch_bounds__(256) void prepack_conv_f16(const unsigned short *src, unsigned short *dst, int I,
                                                        int KH, int KW, size_t total) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  size_t r = i;
  const int ob = (int)(r % 16);
  r /= 16;
  const int ib = (int)(r % 16);
  r /= 16;
  const int y = (int)(r % KW);
  r /= KW;
  const int x = (int)(r % KH);
  r /= KH;
  const int ic = (int)(r % (I / 16));
  const int oc = (int)(r / (I / 16));
  dst[i] = src[(((size_t)(16 * oc + ob) * I + 16 * ic + ib) * KH + x) * KW + y];
}

int launched(const char *what) {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace
}  // namespace unit

extern "C" int unit_pack_nchwc(const void *src, void *dst, int32_t N, int32_t C, int32_t H, int32_t W, int32_t cb,
                               int32_t elem_size, unit_stream_t stream) {
  return unit::nchwc<true>(src, dst, N, C, H, W, cb, elem_size, static_cast<hipStream_t>(stream), "unit_pack_nchwc");
}

extern "C" int unit_unpack_nchwc(const void *src, void *dst, int32_t N, int32_t C, int32_t H, int32_t W, int32_t cb,
                                 int32_t elem_size, unit_stream_t stream) {
  return unit::nchwc<false>(src, dst, N, C, H, W, cb, elem_size, static_cast<hipStream_t>(stream),
                            "unit_unpack_nchwc");
}

extern "C" int unit_prepack_conv_weight_s8(const void *src, void *dst, int32_t O, int32_t I, int32_t KH, int32_t KW,
                                           int32_t cb, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_prepack_conv_weight_s8";
  if (!src || !dst) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (O <= 0 || I <= 0 || KH <= 0 || KW <= 0) return fail(UNIT_E_ARG, "%s: O, I, KH, KW must be positive", what);
  if (cb != 16 && cb != 4) return fail(UNIT_E_ARG, "%s: cb must be 16 or 4 (got %d)", what, cb);
  const int cc = ceil_div(I, cb), ko = ceil_div(O, 16);
  const size_t words = (size_t)ko * cc * KH * KW * (cb / 4) * 16;
  if (!fits(words * 4) || !fits((size_t)O * I * KH * KW)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(prepack_conv_s8, dim3((unsigned)((words + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const signed char *>(src),
                     static_cast<int *>(dst), O, I, KH, KW, cb, cc, words);
  return launched(what);
}

extern "C" int unit_prepack_dense_weight_s8(const void *src, void *dst, int32_t N, int32_t K, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_prepack_dense_weight_s8";
  if (!src || !dst) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (N <= 0 || K <= 0 || N % 128 || K % 4)
    return fail(UNIT_E_ARG, "%s: N must be a positive multiple of 128 and K of 4 (got %d, %d)", what, N, K);
  const size_t words = (size_t)N * K / 4;
  if (!fits(words * 4)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(prepack_dense_s8, dim3((unsigned)((words + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const int *>(src), static_cast<int *>(dst), K / 4,
                     words);
  return launched(what);
}

extern "C" int unit_prepack_conv_weight_f16(const void *src, void *dst, int32_t O, int32_t I, int32_t KH, int32_t KW,
                                            unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_prepack_conv_weight_f16";
  if (!src || !dst) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (O <= 0 || I <= 0 || KH <= 0 || KW <= 0 || O % 16 || I % 16)
    return fail(UNIT_E_ARG, "%s: O and I must be positive multiples of 16 (got %d, %d)", what, O, I);
  const size_t total = (size_t)O * I * KH * KW;
  if (!fits(total * 2)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(prepack_conv_f16, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const unsigned short *>(src),
                     static_cast<unsigned short *>(dst), I, KH, KW, total);
  return launched(what);
}
