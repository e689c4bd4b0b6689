/*
 * CPU oracle for the tensorized u8 x s8 -> i32 conv2d / dense path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the arithmetic the
 * reference generates through TVM for x86 VNNI.  It is the checker for the HIP
 * kernels and the timed CPU baseline; nothing in the shipped package may link,
 * import or call it.
 *
 * Every function cites the reference file:line it restates (paths relative to the
 * reference tree).
 */
#ifndef UNIT_ORACLE_H
#define UNIT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 1 if the host executes AVX-512 VNNI (vpdpbusd), else 0. */
int oracle_has_vnni(void);

/* Threads the *_mt entry points will use when nthreads <= 0. */
int oracle_default_threads(void);

/* ---- deterministic counter-based RNG (splitmix64), shared with the numpy twin ---- */
/* byte i of the stream `seed` = low 8 bits of splitmix64(seed * 0x9E3779B97F4A7C15 + i) */
void oracle_fill_u8(uint8_t *dst, size_t n, uint64_t seed);
void oracle_fill_s8(int8_t *dst, size_t n, uint64_t seed);

/* ---- a1: the VNNI stencil (python/tensorizer/intrinsics/pattern.py:3-16) ----
 * acc[x] += sum_{r<4} (i32)(u8)a[4x+r] * (i32)(s8)b[4x+r],  x < 16, wrapping mod 2^32.
 * `scalar` is the closed form; `hw` executes the real vpdpbusd (poc/vnni/poc.cc:22-26)
 * and returns 0, or returns -1 without touching acc when the host lacks VNNI. */
void oracle_vpdpbusd_scalar(int32_t acc[16], const uint8_t a[64], const int8_t b[64]);
int oracle_vpdpbusd_hw(int32_t acc[16], const uint8_t a[64], const int8_t b[64]);

/* ---- a2: int8 conv2d in NCHW[cb]c (apps/cpu/kernel/conv2d.py:18-30,50-51;
 * closed form apps/cpu/kernel/conv3d.py:60-64) ----
 * data   u8  (N, C/cb, H, W, cb)               cb in {4, 16}
 * weight s8  (K/16, C/cb, KH, KW, cb/4, 16, 4)
 * out    i32 (N, K/16, OH, OW, 16)
 * OH = (H + pt + pb - dh*(KH-1) - 1)/sh + 1, same for OW.  Padding is zero padding of
 * the u8 data (the reference pads in a separate stage and logs pre-padded shapes,
 * cpu-shapes.log:377).  C and K here are the padded channel counts (C % cb == 0,
 * K % 16 == 0).  Returns 0, or -1 on bad arguments. */
typedef struct {
  int N, C, H, W, K, KH, KW;
  int sh, sw;
  int pt, pl, pb, pr;
  int dh, dw;
  int cb;
} oracle_conv_t;

int oracle_conv_out_hw(const oracle_conv_t *p, int *OH, int *OW);

/* scalar int32 loops straight from the closed form */
int oracle_conv2d_nchwc_scalar(const oracle_conv_t *p, const uint8_t *data, const int8_t *weight,
                               int32_t *out);
/* vpdpbusd with the reference's loop nest (python/tensorizer/intrinsics/cpu.py:91-183):
 * parallel fused (n, ko, oh), reduction (ci, kh, kw, e), <=28 unrolled ow accumulators,
 * one 16-lane x 4 stencil per (pixel, e).  Falls back to the scalar loops without VNNI.
 * nthreads <= 0 -> all cores in the affinity mask. */
int oracle_conv2d_nchwc_vnni(const oracle_conv_t *p, const uint8_t *data, const int8_t *weight,
                             int32_t *out, int nthreads);

/* ---- a3: int8 dense (apps/cpu/kernel/int8-gemm.py:9-16; relay form
 * apps/cpu/relay/int8-gemm.py:14-16) ----
 * a  u8 (M, K) row-major;  wp s8 (N/128, K/4, 128, 4) with wp[n/128][k/4][n%128][k%4] = W[n][k];
 * c  i32 (M, N) = a . W^T.   N % 128 == 0, K % 4 == 0.
 * The packed index order is this build's reading of the placeholder shape; the
 * reference never checks values through it (parity unpinned for the index order, pinned
 * for the logical product a . W^T). */
int oracle_dense_scalar(const uint8_t *a, const int8_t *wp, int32_t *c, int M, int N, int K);
int oracle_dense_vnni(const uint8_t *a, const int8_t *wp, int32_t *c, int M, int N, int K,
                      int nthreads);

/* host vpdpbusd peak in the style of poc/vnni/micro.cc:16-51: 8 independent chains,
 * `iters` rounds on `nthreads` threads; returns giga-vpdpbusd per second (x128 = Gop/s). */
double oracle_vnni_peak(long iters, int nthreads);

#ifdef __cplusplus
}
#endif
#endif
