/*
 * CPU oracle, AVX-512 VNNI half.  TEST INFRASTRUCTURE ONLY: see unit_oracle.h.
 * Built with -mavx512f -mavx512bw -mavx512vnni; entered only after the CPUID check
 * in unit_oracle.c.
 *
 * Instruction: llvm.x86.avx512.vpdpbusd.512 as emitted at
 * python/tensorizer/intrinsics/cpu.py:42-49,189-193 (C form: poc/vnni/poc.cc:22-26).
 * In the conv / dense stencil the u8 operand is 4 activation bytes broadcast to all
 * 16 lanes (cpu.py:30-33) and the s8 operand is 64 contiguous weight bytes
 * (16 output channels x 4 input channels).
 */
#include <immintrin.h>
#include <stdlib.h>
#include <string.h>
#include <sys/time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#include "unit_oracle.h"

void oracle_vnni_impl_vpdpbusd(int32_t acc[16], const uint8_t a[64], const int8_t b[64]) {
  __m512i va = _mm512_loadu_si512((const void *)a);
  __m512i vb = _mm512_loadu_si512((const void *)b);
  __m512i vc = _mm512_loadu_si512((const void *)acc);
  _mm512_storeu_si512((void *)acc, _mm512_dpbusd_epi32(vc, va, vb));
}

static inline int load_i32(const uint8_t *p) {
  int v;
  memcpy(&v, p, 4);
  return v;
}

/* One output row segment of T pixels x 16 output channels: T zmm accumulators, the
 * reduction (ci, kh, kw, e) outside the unrolled pixel loop (cpu.py:180-183 order:
 * fusion, simple, reduction, unroll, stencil). */
static inline __attribute__((always_inline)) void conv_row_tile(
    const int T, const oracle_conv_t *p, int Hp, int Wp, const uint8_t *A, const int8_t *Wt,
    int32_t *o, int n, int ko, int oh, int ow0) {
  const int cb = p->cb, Cc = p->C / cb, E = cb / 4;
  __m512i acc[28];
  int t, ci, kh, kw, e;
  for (t = 0; t < T; ++t) acc[t] = _mm512_setzero_si512();
  for (ci = 0; ci < Cc; ++ci)
    for (kh = 0; kh < p->KH; ++kh)
      for (kw = 0; kw < p->KW; ++kw) {
        const uint8_t *ap = A + ((((size_t)n * Cc + ci) * Hp + oh * p->sh + kh * p->dh) * Wp +
                                 ow0 * p->sw + kw * p->dw) * cb;
        const int8_t *wq = Wt + ((((size_t)ko * Cc + ci) * p->KH + kh) * p->KW + kw) * (size_t)E * 64;
        for (e = 0; e < E; ++e) {
          __m512i wv = _mm512_loadu_si512((const void *)(wq + e * 64));
          for (t = 0; t < T; ++t)
            acc[t] = _mm512_dpbusd_epi32(
                acc[t], _mm512_set1_epi32(load_i32(ap + (size_t)t * p->sw * cb + 4 * e)), wv);
        }
      }
  for (t = 0; t < T; ++t) _mm512_storeu_si512((void *)(o + 16 * t), acc[t]);
}

#define ROW_TILE_CASE(T)                                         \
  case T:                                                        \
    conv_row_tile(T, p, Hp, Wp, A, Wt, o, n, ko, oh, ow);        \
    break;

void oracle_vnni_impl_conv(const oracle_conv_t *p, int OH, int OW, int Hp, int Wp,
                           const uint8_t *A, const int8_t *Wt, int32_t *out, int nthreads) {
  const int Ko = p->K / 16;
  const long rows = (long)p->N * Ko * OH;
  long r;
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#else
  (void)nthreads;
#endif
#pragma omp parallel for schedule(static) num_threads(nthreads)
  for (r = 0; r < rows; ++r) {
    int oh = (int)(r % OH), ko = (int)((r / OH) % Ko), n = (int)(r / ((long)OH * Ko));
    int ow = 0;
    while (ow < OW) {
      int left = OW - ow, T;
      int32_t *o = out + ((((size_t)n * Ko + ko) * OH + oh) * OW + ow) * 16;
      /* widest tile that fits, <= 28 accumulators (looptiler.py:22 max_unroll=32) */
      if (left >= 28) T = 28;
      else if (left >= 16) T = 16;
      else if (left >= 14) T = 14;
      else if (left >= 8) T = 8;
      else if (left >= 7) T = 7;
      else if (left >= 4) T = 4;
      else if (left >= 2) T = 2;
      else T = 1;
      switch (T) {
        ROW_TILE_CASE(28)
        ROW_TILE_CASE(16)
        ROW_TILE_CASE(14)
        ROW_TILE_CASE(8)
        ROW_TILE_CASE(7)
        ROW_TILE_CASE(4)
        ROW_TILE_CASE(2)
        ROW_TILE_CASE(1)
      }
      ow += T;
    }
  }
}

/* TM rows x 32 output columns (2 zmm): wp[n/128][k/4][n%128][k%4], 64 bytes = 16 n x 4 k */
static inline __attribute__((always_inline)) void dense_tile(const int TM, const uint8_t *a,
                                                             const int8_t *wp, int32_t *c, int N,
                                                             int K, int m0, int n0) {
  __m512i acc0[14], acc1[14];
  const int8_t *w = wp + ((size_t)(n0 / 128) * (K / 4)) * 512 + (size_t)(n0 % 128) * 4;
  int t, kg;
  for (t = 0; t < TM; ++t) {
    acc0[t] = _mm512_setzero_si512();
    acc1[t] = _mm512_setzero_si512();
  }
  for (kg = 0; kg < K / 4; ++kg) {
    __m512i w0 = _mm512_loadu_si512((const void *)(w + (size_t)kg * 512));
    __m512i w1 = _mm512_loadu_si512((const void *)(w + (size_t)kg * 512 + 64));
    for (t = 0; t < TM; ++t) {
      __m512i av = _mm512_set1_epi32(load_i32(a + (size_t)(m0 + t) * K + 4 * kg));
      acc0[t] = _mm512_dpbusd_epi32(acc0[t], av, w0);
      acc1[t] = _mm512_dpbusd_epi32(acc1[t], av, w1);
    }
  }
  for (t = 0; t < TM; ++t) {
    _mm512_storeu_si512((void *)(c + (size_t)(m0 + t) * N + n0), acc0[t]);
    _mm512_storeu_si512((void *)(c + (size_t)(m0 + t) * N + n0 + 16), acc1[t]);
  }
}

#define DENSE_TILE_CASE(T)                      \
  case T:                                       \
    dense_tile(T, a, wp, c, N, K, m0, n0);      \
    break;

void oracle_vnni_impl_dense(const uint8_t *a, const int8_t *wp, int32_t *c, int M, int N, int K,
                            int nthreads) {
  const int TMAX = 14;
  const long mt = (M + TMAX - 1) / TMAX, nt = N / 32, tiles = mt * nt;
  long i;
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#else
  (void)nthreads;
#endif
#pragma omp parallel for schedule(static) num_threads(nthreads)
  for (i = 0; i < tiles; ++i) {
    /* n fastest inside a thread's chunk so the A rows stay in L1/L2 */
    int m0 = (int)(i / nt) * TMAX, n0 = (int)(i % nt) * 32;
    int TM = M - m0 < TMAX ? M - m0 : TMAX;
    switch (TM) {
      DENSE_TILE_CASE(14)
      DENSE_TILE_CASE(13)
      DENSE_TILE_CASE(12)
      DENSE_TILE_CASE(11)
      DENSE_TILE_CASE(10)
      DENSE_TILE_CASE(9)
      DENSE_TILE_CASE(8)
      DENSE_TILE_CASE(7)
      DENSE_TILE_CASE(6)
      DENSE_TILE_CASE(5)
      DENSE_TILE_CASE(4)
      DENSE_TILE_CASE(3)
      DENSE_TILE_CASE(2)
      DENSE_TILE_CASE(1)
    }
  }
}

/* poc/vnni/micro.cc:16-51: 8 independent vpdpbusd chains per thread */
double oracle_vnni_impl_peak(long iters, int nthreads) {
  struct timeval t0, t1;
  volatile int sink = 0;
  double sec;
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#else
  nthreads = 1;
#endif
  gettimeofday(&t0, NULL);
#pragma omp parallel num_threads(nthreads)
  {
    __m512i a = _mm512_set1_epi8(3), b = _mm512_set1_epi8(-2);
    __m512i c0 = _mm512_setzero_si512(), c1 = c0, c2 = c0, c3 = c0, c4 = c0, c5 = c0, c6 = c0, c7 = c0;
    long i;
    for (i = 0; i < iters; ++i) {
      c0 = _mm512_dpbusd_epi32(c0, a, b);
      c1 = _mm512_dpbusd_epi32(c1, a, b);
      c2 = _mm512_dpbusd_epi32(c2, a, b);
      c3 = _mm512_dpbusd_epi32(c3, a, b);
      c4 = _mm512_dpbusd_epi32(c4, a, b);
      c5 = _mm512_dpbusd_epi32(c5, a, b);
      c6 = _mm512_dpbusd_epi32(c6, a, b);
      c7 = _mm512_dpbusd_epi32(c7, a, b);
      __asm__ volatile("" : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3), "+v"(c4), "+v"(c5), "+v"(c6), "+v"(c7));
    }
    c0 = _mm512_add_epi32(_mm512_add_epi32(c0, c1), _mm512_add_epi32(c2, c3));
    c4 = _mm512_add_epi32(_mm512_add_epi32(c4, c5), _mm512_add_epi32(c6, c7));
    sink += _mm512_reduce_add_epi32(_mm512_add_epi32(c0, c4));
  }
  gettimeofday(&t1, NULL);
  (void)sink;
  sec = (double)(t1.tv_sec - t0.tv_sec) + 1e-6 * (double)(t1.tv_usec - t0.tv_usec);
  return 8.0 * (double)iters * (double)nthreads / sec * 1e-9;
}
