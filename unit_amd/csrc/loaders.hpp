// Operand-tile loaders for mma_kernel: each stages ROWS x BKB reduction bytes per pipeline step,
// global -> registers (fetch) -> swizzled LDS rows (commit).
#pragma once
#include "mma_core.hpp"

namespace unit {

__device__ __forceinline__ v4i zero4() { return v4i{0, 0, 0, 0}; }

// ------------------------------------------------------------------------------------------
// Rows that are K-contiguous in memory: GEMM A (M, K) u8 / f16 and W (N, K) s8.
// Thread t owns chunk column t % CPR of rows t / CPR + i * NT / CPR: 8 (or 4) consecutive lanes
// read one whole 128-byte (64-byte) row segment.
// ------------------------------------------------------------------------------------------
template <int ROWS, int BKB, int NT, bool XOR80>
struct RowMajorLoader {
  struct Params {
    const char *base;
    int rows;    // valid rows
    int ld;      // row pitch in bytes
    int kbytes;  // valid reduction bytes per row (multiple of 16)
  };
  static constexpr bool kNeedsSync = false;
  static constexpr int CPR = BKB / 16, RPP = NT / CPR, NCH = ROWS / RPP;
  static_assert(NT % CPR == 0 && ROWS % RPP == 0 && RPP % 16 == 0, "row-major loader shape");

  v4i r[NCH];
  u32 off[NCH];
  const char *base;
  int kleft;   // kbytes - c*16: chunk of stage kt is valid iff kt*BKB < kleft
  int ldsoff;  // LDS offset of chunk 0

  __device__ __forceinline__ void init(const Params &p, int row0, int t, char *) {
    const int c = t % CPR, rr = t / CPR;
    base = p.base + c * 16;
    kleft = p.kbytes - c * 16;
    ldsoff = lds_off<BKB>(rr, c);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      int row = row0 + rr + i * RPP;
      row = row < p.rows ? row : p.rows - 1;
      off[i] = (u32)row * (u32)p.ld;
    }
  }
  __device__ __forceinline__ void fetch(int kt) {
    const int kb = kt * BKB;
    const bool ok = kb < kleft;
#pragma unroll
    for (int i = 0; i < NCH; ++i)
      r[i] = ok ? *reinterpret_cast<const v4i *>(base + off[i] + kb) : zero4();
  }
  __device__ __forceinline__ void commit(char *tile) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      v4i v = r[i];
      if (XOR80) v ^= (int)0x80808080;
      *reinterpret_cast<v4i *>(tile + ldsoff + i * RPP * BKB) = v;
    }
  }
};

// ------------------------------------------------------------------------------------------
// s8 weights in the reference's VNNI pre-pack: [n / NB][kg][n % NB][4] with kg = k / 4.
//   NB = 128: dense   (N/128, K/4, 128, 4)
//   NB = 16 : conv    (K/16, C/cb, KH, KW, cb/4, 16, 4)  (kg runs over ci, kh, kw, e)
// A thread loads, for 4 consecutive n, the 4 k-groups of one 16-byte reduction chunk (4 x 16
// bytes), transposes the 4x4 dwords in registers (free) and writes one 16-byte LDS chunk per n.
// ------------------------------------------------------------------------------------------
template <int ROWS, int BKB, int NT, int NB>
struct VnniLoader {
  struct Params {
    const char *base;
    int rows;      // valid n (multiple of 16)
    int kg_total;  // k-groups per n
  };
  static constexpr bool kNeedsSync = false;
  static constexpr int CPR = BKB / 16, QUADS = ROWS / 4, UNITS = QUADS * CPR;
  static constexpr int UPT = (UNITS + NT - 1) / NT;
  static constexpr bool kAllActive = UNITS % NT == 0;  // else UNITS < NT: threads >= UNITS idle
  static_assert(kAllActive || UNITS < NT, "vnni loader shape");

  v4i r[UPT][4];
  const char *ptr[UPT];  // address of k-group 4*c of the thread's 4 n
  int cidx[UPT];         // chunk column inside the stage
  int lrow[UPT];         // first LDS row (n quad)
  int kg_total;
  int kgstride;          // bytes between consecutive k-groups
  bool active;

  __device__ __forceinline__ void init(const Params &p, int row0, int t, char *) {
    kg_total = p.kg_total;
    kgstride = NB * 4;
    active = kAllActive || t < UNITS;
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int u = i * NT + t;
      const int nq = u % QUADS, c = u / QUADS;
      int n = row0 + nq * 4;
      n = n < p.rows ? n : p.rows - 4;
      cidx[i] = c;
      lrow[i] = nq * 4;
      ptr[i] = p.base + ((size_t)(n / NB) * p.kg_total) * (NB * 4) + (n % NB) * 4 + (size_t)(4 * c) * (NB * 4);
    }
  }
  __device__ __forceinline__ void fetch(int kt) {
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int kg0 = (kt * CPR + cidx[i]) * 4;
      const char *q = ptr[i] + (size_t)(kt * CPR * 4) * kgstride;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        r[i][d] = (active && kg0 + d < kg_total) ? *reinterpret_cast<const v4i *>(q + d * kgstride) : zero4();
    }
  }
  __device__ __forceinline__ void commit(char *tile) {
    if (!active) return;
#pragma unroll
    for (int i = 0; i < UPT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v4i v = {r[i][0][j], r[i][1][j], r[i][2][j], r[i][3][j]};
        *reinterpret_cast<v4i *>(tile + lds_off<BKB>(lrow[i] + j, cidx[i])) = v;
      }
  }
};

// ------------------------------------------------------------------------------------------
// fp16 operand stored reduction-major ("K x N"): GEMM B (K, N) row-major, and the conv weight
// (K/16, C/16, KH, KW, 16 in, 16 out).  address(k, n) = (n / NBLK) * blk_stride + k * row_stride
// + (n % NBLK) * 2.  A thread loads an 8 (k) x 4 (n) patch as 8 x 8 bytes, transposes it with
// v_perm_b32 and writes one 16-byte chunk (8 k) per n.
// ------------------------------------------------------------------------------------------
template <int ROWS, int BKB, int NT>
struct KMajorF16Loader {
  struct Params {
    const char *base;
    int rows;          // valid n (multiple of 4)
    int ktotal;        // valid k (multiple of 8)
    int nblk;          // n per block (GEMM: >= N)
    size_t blk_stride; // bytes between n-blocks
    int row_stride;    // bytes between consecutive k
  };
  static constexpr bool kNeedsSync = false;
  static constexpr int CPR = BKB / 16, QUADS = ROWS / 4, UNITS = QUADS * CPR;
  static constexpr int UPT = (UNITS + NT - 1) / NT;
  static constexpr bool kAllActive = UNITS % NT == 0;  // else UNITS < NT: threads >= UNITS idle
  static_assert(kAllActive || UNITS < NT, "k-major loader shape");

  v2i r[UPT][8];
  const char *ptr[UPT];
  int cidx[UPT], lrow[UPT];
  int ktotal, row_stride;
  bool active;

  __device__ __forceinline__ void init(const Params &p, int row0, int t, char *) {
    ktotal = p.ktotal;
    row_stride = p.row_stride;
    active = kAllActive || t < UNITS;
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int u = i * NT + t;
      const int nq = u % QUADS, c = u / QUADS;
      int n = row0 + nq * 4;
      n = n < p.rows ? n : p.rows - 4;
      cidx[i] = c;
      lrow[i] = nq * 4;
      ptr[i] = p.base + (size_t)(n / p.nblk) * p.blk_stride + (size_t)(n % p.nblk) * 2 +
               (size_t)(8 * c) * p.row_stride;
    }
  }
  __device__ __forceinline__ void fetch(int kt) {
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int k0 = (kt * CPR + cidx[i]) * 8;
      const char *q = ptr[i] + (size_t)(kt * CPR * 8) * row_stride;
      const bool ok = active && k0 < ktotal;  // ktotal % 8 == 0: a chunk is all valid or all padding
#pragma unroll
      for (int kk = 0; kk < 8; ++kk)
        r[i][kk] = ok ? *reinterpret_cast<const v2i *>(q + (size_t)kk * row_stride) : v2i{0, 0};
    }
  }
  __device__ __forceinline__ void commit(char *tile) {
    if (!active) return;
#pragma unroll
    for (int i = 0; i < UPT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // halves j of rows 2p and 2p+1 -> dword p
        const u32 sel = (j & 1) ? 0x07060302u : 0x05040100u;
        v4i v;
#pragma unroll
        for (int p = 0; p < 4; ++p)
          v[p] = (int)__builtin_amdgcn_perm((u32)r[i][2 * p + 1][j >> 1], (u32)r[i][2 * p][j >> 1], sel);
        *reinterpret_cast<v4i *>(tile + lds_off<BKB>(lrow[i] + j, cidx[i])) = v;
      }
  }
};

// ------------------------------------------------------------------------------------------
// Convolution data gathered on the fly (implicit im2col): row = output pixel, reduction =
// taps (ci, kh, kw) in memory order of the weight tensor, each tap contributing TAPB bytes of
// one input pixel's channel block:
//   TAPB = 16: u8 NCHW16c   (one 16-byte chunk per tap)
//   TAPB = 4 : u8 NCHW4c    (four taps per chunk, gathered as dwords)
//   TAPB = 32: f16 NCHW16c  (two chunks per tap)
// Consecutive lanes own consecutive output pixels, so for stride 1 a wave reads 1 KiB of
// contiguous input per tap.  Taps outside the image (zero padding) and beyond the last tap are
// staged as zeros (0x80 after the u8 -> s8 shift, i.e. the value of a zero pixel).
// A table tap -> (byte offset, dilated kh, kw) is built once per workgroup in LDS.
// ------------------------------------------------------------------------------------------
struct ConvGeom {
  int N, H, W, OH, OW;
  int KH, KW, sh, sw, pt, pl, dh, dw;
  int npix;    // N * OH * OW
  int ntaps;   // (C / cb) * KH * KW
  int ntab;    // table entries (ntaps rounded up to whole pipeline stages)
  u32 img_bytes;  // bytes per image
};

template <int ROWS, int BKB, int NT, int TAPB, bool XOR80>
struct ConvPixelLoader {
  struct Params {
    const char *base;
    ConvGeom g;
  };
  static constexpr bool kNeedsSync = true;
  static constexpr int CPR = BKB / 16;
  static constexpr int PPT = ROWS > NT ? ROWS / NT : 1;   // pixels per thread
  static constexpr int TPS = NT > ROWS ? NT / ROWS : 1;   // threads sharing a pixel
  static constexpr int NCH = ROWS * CPR / NT;
  static constexpr int CPT = NCH / PPT;                   // chunk columns per thread
  static_assert((ROWS % NT == 0 || NT % ROWS == 0) && NCH >= 1 && CPR % TPS == 0, "pixel loader shape");

  v4i r[NCH];
  int pixoff[PPT];  // byte offset of (n, oh*sh-pt, ow*sw-pl) in the data tensor; INT_MIN/2 = no pixel
  int ih0[PPT], iw0[PPT];
  const char *base;
  const v2i *tab;
  int H, W, tq, prow;

  __device__ __forceinline__ void init(const Params &p, int row0, int t, char *aux) {
    const ConvGeom &g = p.g;
    base = p.base;
    H = g.H;
    W = g.W;
    v2i *tb = reinterpret_cast<v2i *>(aux);
    tab = tb;
    for (int e = t; e < g.ntab; e += NT) {
      v2i ent;
      if (e < g.ntaps) {
        const int kw = e % g.KW, rest = e / g.KW, kh = rest % g.KH, ci = rest / g.KH;
        ent[0] = ((ci * g.H + kh * g.dh) * g.W + kw * g.dw) * TAPB;
        ent[1] = (kh * g.dh) | ((kw * g.dw) << 16);
      } else {
        ent[0] = 0;
        ent[1] = 0x7fff;  // fails the height test
      }
      tb[e] = ent;
    }
    prow = t % ROWS;
    tq = t / ROWS;
#pragma unroll
    for (int s = 0; s < PPT; ++s) {
      const int m = row0 + prow + s * NT;
      if (m < g.npix) {
        const int n = m / (g.OH * g.OW), rem = m - n * (g.OH * g.OW);
        const int oh = rem / g.OW, ow = rem - oh * g.OW;
        ih0[s] = oh * g.sh - g.pt;
        iw0[s] = ow * g.sw - g.pl;
        pixoff[s] = (int)(n * g.img_bytes) + (ih0[s] * g.W + iw0[s]) * TAPB;
      } else {
        ih0[s] = -0x8000;  // every tap fails the height test
        iw0[s] = 0;
        pixoff[s] = 0;
      }
    }
  }

  __device__ __forceinline__ bool tap_addr(int tap, int s, const char *&src) const {
    const v2i e = tab[tap];
    const int ih = ih0[s] + (e[1] & 0xffff), iw = iw0[s] + (e[1] >> 16);
    src = base + pixoff[s] + e[0];
    return (u32)ih < (u32)H && (u32)iw < (u32)W;
  }

  __device__ __forceinline__ void fetch(int kt) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int s = i % PPT;
      const int g = kt * CPR + (i / PPT) * TPS + tq;  // global chunk index
      const char *src;
      if constexpr (TAPB == 16) {
        r[i] = tap_addr(g, s, src) ? *reinterpret_cast<const v4i *>(src) : zero4();
      } else if constexpr (TAPB == 32) {
        const bool ok = tap_addr(g >> 1, s, src);
        r[i] = ok ? *reinterpret_cast<const v4i *>(src + (g & 1) * 16) : zero4();
      } else {
        static_assert(TAPB == 4 || TAPB == 16 || TAPB == 32, "tap width");
        v4i v;
#pragma unroll
        for (int d = 0; d < 4; ++d) v[d] = tap_addr(4 * g + d, s, src) ? *reinterpret_cast<const int *>(src) : 0;
        r[i] = v;
      }
    }
  }

  __device__ __forceinline__ void commit(char *tile) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      v4i v = r[i];
      if (XOR80) v ^= (int)0x80808080;
      const int row = prow + (i % PPT) * NT;
      *reinterpret_cast<v4i *>(tile + lds_off<BKB>(row, (i / PPT) * TPS + tq)) = v;
    }
  }
};

}  // namespace unit
