/*
 * CPU oracle, scalar half + dispatch.  TEST INFRASTRUCTURE ONLY: see unit_oracle.h.
 * The AVX-512 VNNI half lives in unit_oracle_vnni.c (built with -mavx512vnni) and is
 * entered only after a CPUID check.
 */
#include "unit_oracle.h"

#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* implemented in unit_oracle_vnni.c */
void oracle_vnni_impl_vpdpbusd(int32_t acc[16], const uint8_t a[64], const int8_t b[64]);
void oracle_vnni_impl_conv(const oracle_conv_t *p, int OH, int OW, int Hp, int Wp,
                           const uint8_t *padded, const int8_t *weight, int32_t *out, int nthreads);
void oracle_vnni_impl_dense(const uint8_t *a, const int8_t *wp, int32_t *c, int M, int N, int K,
                            int nthreads);
double oracle_vnni_impl_peak(long iters, int nthreads);

int oracle_has_vnni(void) {
  __builtin_cpu_init();
  return __builtin_cpu_supports("avx512vnni") && __builtin_cpu_supports("avx512f") &&
                 __builtin_cpu_supports("avx512bw")
             ? 1
             : 0;
}

int oracle_default_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---------------------------------------------------------------- RNG */
static inline uint64_t splitmix64(uint64_t x) {
  uint64_t z = x + 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

/* byte i = byte (i % 8), little-endian, of splitmix64(seed * GOLDEN + i / 8) */
void oracle_fill_u8(uint8_t *dst, size_t n, uint64_t seed) {
  const uint64_t base = seed * 0x9E3779B97F4A7C15ull;
  size_t words = n / 8, i;
  for (i = 0; i < words; ++i) {
    uint64_t v = splitmix64(base + i);
    int b;
    for (b = 0; b < 8; ++b) dst[8 * i + b] = (uint8_t)(v >> (8 * b));
  }
  if (n % 8) {
    uint64_t v = splitmix64(base + words);
    size_t b;
    for (b = 0; b < n % 8; ++b) dst[8 * words + b] = (uint8_t)(v >> (8 * b));
  }
}

void oracle_fill_s8(int8_t *dst, size_t n, uint64_t seed) {
  oracle_fill_u8((uint8_t *)dst, n, seed);
}

/* ---------------------------------------------------------------- a1 stencil */
/* python/tensorizer/intrinsics/pattern.py:3-16: c[x] = sum_red i32(a[4x+red]) * i32(b[4x+red]) */
void oracle_vpdpbusd_scalar(int32_t acc[16], const uint8_t a[64], const int8_t b[64]) {
  int x, r;
  for (x = 0; x < 16; ++x) {
    uint32_t s = (uint32_t)acc[x];
    for (r = 0; r < 4; ++r) s += (uint32_t)((int32_t)a[4 * x + r] * (int32_t)b[4 * x + r]);
    acc[x] = (int32_t)s;
  }
}

int oracle_vpdpbusd_hw(int32_t acc[16], const uint8_t a[64], const int8_t b[64]) {
  if (!oracle_has_vnni()) return -1;
  oracle_vnni_impl_vpdpbusd(acc, a, b);
  return 0;
}

/* ---------------------------------------------------------------- a2 conv */
static int conv_args_ok(const oracle_conv_t *p) {
  if (!p) return 0;
  if (p->cb != 4 && p->cb != 16) return 0;
  if (p->N <= 0 || p->C <= 0 || p->H <= 0 || p->W <= 0 || p->K <= 0) return 0;
  if (p->KH <= 0 || p->KW <= 0 || p->sh <= 0 || p->sw <= 0 || p->dh <= 0 || p->dw <= 0) return 0;
  if (p->pt < 0 || p->pl < 0 || p->pb < 0 || p->pr < 0) return 0;
  if (p->C % p->cb || p->K % 16) return 0;
  return 1;
}

int oracle_conv_out_hw(const oracle_conv_t *p, int *OH, int *OW) {
  int eh, ew;
  if (!conv_args_ok(p)) return -1;
  eh = p->H + p->pt + p->pb - p->dh * (p->KH - 1) - 1;
  ew = p->W + p->pl + p->pr - p->dw * (p->KW - 1) - 1;
  if (eh < 0 || ew < 0) return -1;
  *OH = eh / p->sh + 1;
  *OW = ew / p->sw + 1;
  return 0;
}

/* zero-padded copy of the data tensor, (N, C/cb, Hp, Wp, cb); caller frees */
static uint8_t *pad_data(const oracle_conv_t *p, const uint8_t *data, int *Hp, int *Wp) {
  int Cc = p->C / p->cb, hp = p->H + p->pt + p->pb, wp = p->W + p->pl + p->pr;
  size_t planes = (size_t)p->N * Cc, i;
  uint8_t *buf = (uint8_t *)calloc(planes * hp * wp * p->cb + 64, 1);
  int h;
  if (!buf) return NULL;
  for (i = 0; i < planes; ++i)
    for (h = 0; h < p->H; ++h)
      memcpy(buf + ((i * hp + h + p->pt) * wp + p->pl) * p->cb,
             data + ((i * p->H + h) * (size_t)p->W) * p->cb, (size_t)p->W * p->cb);
  *Hp = hp;
  *Wp = wp;
  return buf;
}

/* apps/cpu/kernel/conv3d.py:60-64 (2-D case): out[n,ko,oh,ow,kb] =
 *   sum_{ci,kh,kw,e,i} i32(A[n,ci,sh*oh+dh*kh,sw*ow+dw*kw,4e+i]) * i32(W[ko,ci,kh,kw,e,kb,i]) */
int oracle_conv2d_nchwc_scalar(const oracle_conv_t *p, const uint8_t *data, const int8_t *weight,
                               int32_t *out) {
  int OH, OW, Hp, Wp, Cc, Ko, E, cb;
  uint8_t *A;
  int n, ko, oh, ow, kb, ci, kh, kw, e, i;
  if (oracle_conv_out_hw(p, &OH, &OW)) return -1;
  A = pad_data(p, data, &Hp, &Wp);
  if (!A) return -1;
  cb = p->cb;
  Cc = p->C / cb;
  Ko = p->K / 16;
  E = cb / 4;
  for (n = 0; n < p->N; ++n)
    for (ko = 0; ko < Ko; ++ko)
      for (oh = 0; oh < OH; ++oh)
        for (ow = 0; ow < OW; ++ow) {
          int32_t *o = out + ((((size_t)n * Ko + ko) * OH + oh) * OW + ow) * 16;
          for (kb = 0; kb < 16; ++kb) {
            uint32_t s = 0;
            for (ci = 0; ci < Cc; ++ci)
              for (kh = 0; kh < p->KH; ++kh)
                for (kw = 0; kw < p->KW; ++kw) {
                  const uint8_t *ap =
                      A + ((((size_t)n * Cc + ci) * Hp + oh * p->sh + kh * p->dh) * Wp +
                           ow * p->sw + kw * p->dw) * cb;
                  const int8_t *wq =
                      weight + ((((size_t)ko * Cc + ci) * p->KH + kh) * p->KW + kw) * (size_t)E * 64;
                  for (e = 0; e < E; ++e)
                    for (i = 0; i < 4; ++i)
                      s += (uint32_t)((int32_t)ap[4 * e + i] * (int32_t)wq[(e * 16 + kb) * 4 + i]);
                }
            o[kb] = (int32_t)s;
          }
        }
  free(A);
  return 0;
}

int oracle_conv2d_nchwc_vnni(const oracle_conv_t *p, const uint8_t *data, const int8_t *weight,
                             int32_t *out, int nthreads) {
  int OH, OW, Hp, Wp;
  uint8_t *A;
  if (!oracle_has_vnni()) return oracle_conv2d_nchwc_scalar(p, data, weight, out);
  if (oracle_conv_out_hw(p, &OH, &OW)) return -1;
  if (p->pt || p->pl || p->pb || p->pr) {
    A = pad_data(p, data, &Hp, &Wp);
    if (!A) return -1;
    oracle_vnni_impl_conv(p, OH, OW, Hp, Wp, A, weight, out, nthreads);
    free(A);
  } else {
    oracle_vnni_impl_conv(p, OH, OW, p->H, p->W, data, weight, out, nthreads);
  }
  return 0;
}

/* ---------------------------------------------------------------- a3 dense */
int oracle_dense_scalar(const uint8_t *a, const int8_t *wp, int32_t *c, int M, int N, int K) {
  int m, n, k;
  if (M <= 0 || N <= 0 || K <= 0 || N % 128 || K % 4) return -1;
  for (m = 0; m < M; ++m)
    for (n = 0; n < N; ++n) {
      const int8_t *w = wp + ((size_t)(n / 128) * (K / 4)) * 512 + (size_t)(n % 128) * 4;
      uint32_t s = 0;
      for (k = 0; k < K; ++k)
        s += (uint32_t)((int32_t)a[(size_t)m * K + k] * (int32_t)w[(size_t)(k / 4) * 512 + k % 4]);
      c[(size_t)m * N + n] = (int32_t)s;
    }
  return 0;
}

int oracle_dense_vnni(const uint8_t *a, const int8_t *wp, int32_t *c, int M, int N, int K,
                      int nthreads) {
  if (M <= 0 || N <= 0 || K <= 0 || N % 128 || K % 4) return -1;
  if (!oracle_has_vnni()) return oracle_dense_scalar(a, wp, c, M, N, K);
  oracle_vnni_impl_dense(a, wp, c, M, N, K, nthreads);
  return 0;
}

double oracle_vnni_peak(long iters, int nthreads) {
  if (!oracle_has_vnni()) return 0.0;
  return oracle_vnni_impl_peak(iters, nthreads);
}
