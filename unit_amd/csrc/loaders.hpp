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
// TAIL = false (all three k-contiguous loaders): the reduction is a whole number of stages, so no
// chunk lies past its end and the select instructions that zero such chunks (one per staged
// dword) are left out.
// ------------------------------------------------------------------------------------------
template <int ROWS, int BKB, int NT, bool XOR80, int PF = 1, bool TAIL = true>
struct RowMajorLoader {
  struct Params {
    const char *base;
    int rows;    // valid rows
    int ld;      // row pitch in bytes
    int kbytes;  // valid reduction bytes per row (multiple of 16)
  };
  static constexpr bool kNeedsSync = false;
  static constexpr int kPF = PF;
  static constexpr int CPR = BKB / 16, RPP = NT / CPR, NCH = ROWS / RPP;
  static constexpr int kLoads = NCH;  // global loads per thread and stage
  static_assert(NT % CPR == 0 && ROWS % RPP == 0 && RPP % 16 == 0, "row-major loader shape");

  v4i r[PF][NCH];
  u32 off[NCH];
  bool okm[PF];  // stage in the slot lies inside the reduction (else it is staged as zeros)
  const char *base;
  int coff;    // byte offset of the thread's chunk column inside a stage
  int kleft;   // kbytes - c*16: chunk of stage kt is valid iff kt*BKB < kleft
  int ldsoff;  // LDS offset of chunk 0

  __device__ __forceinline__ void init(const Params &p, int row0, int t, char *) {
    const int c = t % CPR, rr = t / CPR;
    base = p.base;
    coff = c * 16;
    kleft = p.kbytes - c * 16;
    ldsoff = lds_off<BKB>(rr, c);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      int row = row0 + rr + i * RPP;
      row = row < p.rows ? row : p.rows - 1;
      off[i] = (u32)row * (u32)p.ld;
    }
  }
  template <int S>
  __device__ __forceinline__ void fetch(int kt) {
    // loads are unconditional (no branches in the pipeline): a chunk past the end of the
    // reduction re-reads the first chunk of the row and is zeroed when it is written to LDS
    const bool ok = !TAIL || kt * BKB < kleft;
    const int kb = ok ? kt * BKB + coff : 0;
    okm[S] = ok;
#pragma unroll
    for (int i = 0; i < NCH; ++i) r[S][i] = *reinterpret_cast<const v4i *>(base + off[i] + kb);
  }
  template <int S>
  __device__ __forceinline__ void commit(char *tile) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      v4i v = (!TAIL || okm[S]) ? r[S][i] : zero4();
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
template <int ROWS, int BKB, int NT, int NB, int PF = 1, bool TAIL = true>
struct VnniLoader {
  struct Params {
    const char *base;
    int rows;      // valid n (multiple of 16)
    int kg_total;  // k-groups per n
  };
  static constexpr bool kNeedsSync = false;
  static constexpr int kPF = PF;
  static constexpr int CPR = BKB / 16, QUADS = ROWS / 4, UNITS = QUADS * CPR;
  static constexpr int UPT = (UNITS + NT - 1) / NT;
  static constexpr bool kAllActive = UNITS % NT == 0;  // else UNITS < NT: threads >= UNITS idle
  static_assert(kAllActive || UNITS < NT, "vnni loader shape");

  v4i r[PF][UPT][4];
  const char *ptr[UPT];  // address of k-group 0 of the thread's 4 n
  int cidx[UPT];         // chunk column inside the stage
  int lrow[UPT];         // first LDS row (n quad)
  int kg_total;
  int kgstride;          // bytes between consecutive k-groups
  int kt_of[PF];         // stage held by each slot (its k-groups are re-checked at commit)
  bool active;

  __device__ __forceinline__ void init(const Params &p, int row0, int t, char *) {
    kg_total = p.kg_total;
    kgstride = NB * 4;
    active = kAllActive || t < UNITS;
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int u = (i * NT + t) % UNITS;  // idle threads shadow a live unit (their loads stay in bounds)
      const int nq = u % QUADS, c = u / QUADS;
      int n = row0 + nq * 4;
      n = n < p.rows ? n : p.rows - 4;
      cidx[i] = c;
      lrow[i] = nq * 4;
      ptr[i] = p.base + ((size_t)(n / NB) * p.kg_total) * (NB * 4) + (n % NB) * 4;
    }
  }
  template <int S>
  __device__ __forceinline__ void fetch(int kt) {
    kt_of[S] = kt;
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int kg0 = (kt * CPR + cidx[i]) * 4;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // unconditional load: a k-group past the end re-reads k-group 0
        const int kg = (!TAIL || kg0 + d < kg_total) ? kg0 + d : 0;
        r[S][i][d] = *reinterpret_cast<const v4i *>(ptr[i] + (size_t)kg * kgstride);
      }
    }
  }
  template <int S>
  __device__ __forceinline__ void commit(char *tile) {
    if (!active) return;
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int left = TAIL ? kg_total - (kt_of[S] * CPR + cidx[i]) * 4 : 4;  // valid k-groups of this chunk
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v4i v = {left > 0 ? r[S][i][0][j] : 0, left > 1 ? r[S][i][1][j] : 0, left > 2 ? r[S][i][2][j] : 0,
                 left > 3 ? r[S][i][3][j] : 0};
        *reinterpret_cast<v4i *>(tile + lds_off<BKB>(lrow[i] + j, cidx[i])) = v;
      }
    }
  }
};

// ------------------------------------------------------------------------------------------
// fp16 operand stored reduction-major ("K x N"): GEMM B (K, N) row-major, and the conv weight
// (K/16, C/16, KH, KW, 16 in, 16 out).  address(k, n) = (n / NBLK) * blk_stride + k * row_stride
// + (n % NBLK) * 2.  A thread loads an 8 (k) x 4 (n) patch as 8 x 8 bytes, transposes it with
// v_perm_b32 and writes one 16-byte chunk (8 k) per n.
// ------------------------------------------------------------------------------------------
template <int ROWS, int BKB, int NT, int PF = 1, bool TAIL = true>
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
  static constexpr int kPF = PF;
  static constexpr int CPR = BKB / 16, QUADS = ROWS / 4, UNITS = QUADS * CPR;
  static constexpr int UPT = (UNITS + NT - 1) / NT;
  static constexpr bool kAllActive = UNITS % NT == 0;  // else UNITS < NT: threads >= UNITS idle
  static constexpr int kLoads = UPT * 8;               // global loads per thread and stage
  static_assert(kAllActive || UNITS < NT, "k-major loader shape");

  v2i r[PF][UPT][8];
  const char *ptr[UPT];
  int cidx[UPT], lrow[UPT];
  int ktotal, row_stride;
  bool okm[PF][UPT];
  bool active;

  __device__ __forceinline__ void init(const Params &p, int row0, int t, char *) {
    ktotal = p.ktotal;
    row_stride = p.row_stride;
    active = kAllActive || t < UNITS;
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int u = (i * NT + t) % UNITS;  // idle threads shadow a live unit
      const int nq = u % QUADS, c = u / QUADS;
      int n = row0 + nq * 4;
      n = n < p.rows ? n : p.rows - 4;
      cidx[i] = c;
      lrow[i] = nq * 4;
      ptr[i] = p.base + (size_t)(n / p.nblk) * p.blk_stride + (size_t)(n % p.nblk) * 2;
    }
  }
  template <int S>
  __device__ __forceinline__ void fetch(int kt) {
#pragma unroll
    for (int i = 0; i < UPT; ++i) {
      const int k0 = (kt * CPR + cidx[i]) * 8;
      const bool ok = !TAIL || k0 < ktotal;  // ktotal % 8 == 0: a chunk is all valid or all padding
      // unconditional loads: a chunk past the end re-reads rows 0..7
      const char *q = ptr[i] + (ok ? (size_t)k0 * row_stride : 0);
      okm[S][i] = ok;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) r[S][i][kk] = *reinterpret_cast<const v2i *>(q + (size_t)kk * row_stride);
    }
  }
  template <int S>
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
          v[p] = (!TAIL || okm[S][i]) ? (int)__builtin_amdgcn_perm((u32)r[S][i][2 * p + 1][j >> 1], (u32)r[S][i][2 * p][j >> 1], sel) : 0;
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
  int c4_steps;  // (C / 4) * KH: k-steps of the direct kernel on 4-channel blocks (one window row each)
  u32 img_bytes;  // bytes per image
  FastDiv by_ohw, by_ow, by_kh, by_kw;  // dividers by output pixels per image, OW, KH, KW
  // depth, for the 3-D convolution (direct kernels only); 1 / 1 / 1 / 1 for 2-D, where
  // by_plane = by_ohw
  int D, KD, sd, nopad;                 // nopad: no zero padding anywhere (every tap of a valid pixel is inside)
  FastDiv by_plane, by_kd;              // dividers by OH * OW, KD
  // bit kh * KW set for every window row kh, when the window is undilated and has at most 31 positions (else 0):
  // the positions of a pixel's window that lie inside the image are then (columns inside) * (these bits of the rows
  // inside), both of them ranges
  u32 row_ones;
};

template <int ROWS, int BKB, int NT, int TAPB, bool XOR80, int PF = 1>
struct ConvPixelLoader {
  struct Params {
    const char *base;
    ConvGeom g;
  };
  static constexpr bool kNeedsSync = true;
  static constexpr int kPF = PF;
  static constexpr int CPR = BKB / 16;
  static constexpr int PPT = ROWS > NT ? ROWS / NT : 1;   // pixels per thread
  static constexpr int TPS = NT > ROWS ? NT / ROWS : 1;   // threads sharing a pixel
  static constexpr int NCH = ROWS * CPR / NT;
  static constexpr int CPT = NCH / PPT;                   // chunk columns per thread
  static_assert((ROWS % NT == 0 || NT % ROWS == 0) && NCH >= 1 && NCH <= 8 && CPR % TPS == 0, "pixel loader shape");

  v4i r[PF][NCH];
  u32 okm[PF];      // bit (4*i + d): dword d of chunk i comes from inside the image
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
        int kw, rest, kh, ci;
        g.by_kw.divmod(e, rest, kw);
        g.by_kh.divmod(rest, ci, kh);
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
        int n, rem, oh, ow;
        g.by_ohw.divmod(m, n, rem);
        g.by_ow.divmod(rem, oh, ow);
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

  // address of a tap's input pixel, or of the tensor start when the tap falls outside the image
  // (zero padding, no pixel, past the last tap): loads stay unconditional and in bounds
  __device__ __forceinline__ bool tap_addr(v2i e, int s, const char *&src) const {
    const int ih = ih0[s] + (e[1] & 0xffff), iw = iw0[s] + (e[1] >> 16);
    const bool ok = (u32)ih < (u32)H && (u32)iw < (u32)W;
    src = base + (ok ? pixoff[s] + e[0] : 0);
    return ok;
  }

  template <int S>
  __device__ __forceinline__ void fetch(int kt) {
    constexpr int TPC = TAPB == 4 ? 4 : 1;  // table entries per chunk
    v2i ent[NCH][TPC];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int g = kt * CPR + (i / PPT) * TPS + tq;  // global chunk index
#pragma unroll
      for (int d = 0; d < TPC; ++d) ent[i][d] = tab[TAPB == 4 ? 4 * g + d : (TAPB == 32 ? g >> 1 : g)];
    }
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int s = i % PPT;
      const int g = kt * CPR + (i / PPT) * TPS + tq;
      const char *src;
      if constexpr (TAPB == 4) {
        v4i v;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          if (tap_addr(ent[i][d], s, src)) m |= 1u << (4 * i + d);
          v[d] = *reinterpret_cast<const int *>(src);
        }
        r[S][i] = v;
      } else {
        static_assert(TAPB == 16 || TAPB == 32, "tap width");
        const bool ok = tap_addr(ent[i][0], s, src);
        if (ok) m |= 0xFu << (4 * i);
        r[S][i] = *reinterpret_cast<const v4i *>(src + ((TAPB == 32 && ok) ? (g & 1) * 16 : 0));
      }
    }
    okm[S] = m;
  }

  template <int S>
  __device__ __forceinline__ void commit(char *tile) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      v4i v;
#pragma unroll
      for (int d = 0; d < 4; ++d) v[d] = (okm[S] >> (4 * i + d)) & 1 ? r[S][i][d] : 0;
      if (XOR80) v ^= (int)0x80808080;
      const int row = prow + (i % PPT) * NT;
      *reinterpret_cast<v4i *>(tile + lds_off<BKB>(row, (i / PPT) * TPS + tq)) = v;
    }
  }
};

}  // namespace unit
