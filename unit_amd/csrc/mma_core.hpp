// Tiled MFMA kernel shared by the int8 / fp16 GEMM and implicit-GEMM convolution entry points.
//
// One workgroup computes a BX x BY tile of  acc[x][y] = sum_k X[x][k] * Y[y][k]  where both
// operand tiles are staged in LDS as rows of BKB reduction *bytes* (K-contiguous), 16-byte
// chunks XOR-swizzled by row.  v_mfma_i32_32x32x32_i8 and v_mfma_f32_32x32x16_f16 both take
// 32 reduction bytes per row per instruction (16 bytes per lane: lanes 0-31 the first chunk,
// lanes 32-63 the second), so the byte-level tiling is identical for the two data types.
//
// X is the first MFMA operand (accumulator rows, spread over registers), Y the second
// (accumulator columns, spread over lanes):  lane l, register r of a 32x32 block hold
//   x = 8*(r/4) + 4*(l/32) + r%4,   y = l%32.
//
// Pipeline: global -> registers (one stage ahead) -> LDS (double buffered) -> fragments (double
// buffered in registers) -> MFMA, one workgroup barrier per stage.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace unit {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned int u32;

// Result stores.  Results are written once and never read back by the kernel that writes them, so they go out as
// agent-scope, non-temporal stores (sc1 nt): sc1 sends the line through the XCD's L2 to memory at once instead of
// leaving it there, dirty, for the write-back at the end of the kernel; nt keeps it from displacing the operands of
// the launches that follow in the memory-side cache.  Measured, 102.8 MB of results: a plain fill 16.4 us on a
// destination that the cache still holds / 17.3 us on a cold one, nt 16.6 / 16.7, sc1 15.1 / 16.0, sc1 nt 15.6 / 15.8;
// the ResNet-50 batch-32 convolution step 0.5415 ms with nt, 0.5777 ms with sc1 alone (its launches find their
// operands evicted: the layers on cold operands take 651 us against 591 us), 0.5324 ms with sc1 nt; the chain of 52
// requantising layers, each reading the previous one's u8 result, 497 us with sc1 nt against 513 us with sc1.
// They are raw buffer stores at a 32-bit byte offset from the tensor's base (tensors stay below 2^31 bytes), the
// form that takes the policy bits as an operand the compiler knows: its hazard and wait-count passes see the stores
// (written as inline assembly they were followed by a write of the data registers inside the store's hazard window).
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
constexpr int kResultPolicy = 16 | 2;  // sc1 | nt
__device__ __forceinline__ __amdgpu_buffer_rsrc_t result_buffer(void *base) {
  return __builtin_amdgcn_make_buffer_rsrc(base, 0, -1, 0x00020000);
}
template <int POLICY = kResultPolicy, class V>
__device__ __forceinline__ void store_result(__amdgpu_buffer_rsrc_t buf, u32 byte_offset, V v) {
  static_assert(sizeof(V) == 16 || sizeof(V) == 4 || sizeof(V) == 2, "results are stored 16, 4 or 2 bytes at a time");
  if constexpr (sizeof(V) == 16)
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), buf, (int)byte_offset, 0, POLICY);
  else if constexpr (sizeof(V) == 4)
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), buf, (int)byte_offset, 0, POLICY);
  else
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), buf, (int)byte_offset, 0, POLICY);
}

// 4-byte-aligned views for gathers whose address is only dword aligned
typedef int v4i_a4 __attribute__((ext_vector_type(4), aligned(4)));

struct OpI8 {
  using acc_t = v16i;
  using out_t = int;
  using out4_t = v4i;
  static constexpr bool kInt = true;
  static __device__ __forceinline__ acc_t mma(v4i x, v4i y, acc_t c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(x, y, c, 0, 0, 0);
  }
};

struct OpF16 {
  using acc_t = v16f;
  using out_t = float;
  using out4_t = v4f;
  static constexpr bool kInt = false;
  static __device__ __forceinline__ acc_t mma(v4i x, v4i y, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, x),
                                                  __builtin_bit_cast(v8h, y), c, 0, 0, 0);
  }
};

// Division of a 31-bit dividend by a runtime constant: q = mulhi(2 n, mul) >> shift with
// shift = ceil(log2 d) and mul = floor(2^(31 + shift) / d) + 1 (2^31 for a power of two), which
// is exact for 0 <= n < 2^31.  Three instructions instead of the ~35 of an integer division;
// pixel and tap indices are decoded this way in kernel prologues and epilogues.
struct FastDiv {
  u32 mul, shift;
  int d;
  __host__ static FastDiv make(int d) {
    FastDiv f;
    f.d = d;
    f.shift = 0;
    while ((1u << f.shift) < (u32)d) ++f.shift;
    f.mul = ((1u << f.shift) == (u32)d) ? 0x80000000u : (u32)((1ull << (31 + f.shift)) / (unsigned long long)d) + 1u;
    return f;
  }
  __device__ __forceinline__ int div(int n) const { return (int)(__umulhi((u32)n << 1, mul) >> shift); }
  __device__ __forceinline__ void divmod(int n, int &q, int &r) const {
    q = div(n);
    r = n - q * d;
  }
};

// XOR mask for the 16-byte chunk index of an LDS row.  Chosen so that any 8 (32 banks) or 16
// (64 banks) consecutive rows reading the same logical chunk land on distinct banks, for rows
// of 128 bytes (8 chunks) and of 64 bytes (4 chunks).
template <int BKB>
__device__ __forceinline__ int swz(int row) {
  if constexpr (BKB == 128) {
    return (row & 7) ^ ((row >> 3) & 1);
  } else {
    static_assert(BKB == 64, "LDS rows are 64 or 128 reduction bytes");
    return ((row >> 1) & 3) ^ ((row >> 3) & 1);
  }
}

template <int BKB>
__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * BKB + ((chunk ^ swz<BKB>(row)) << 4);
}

// FF ("full fragments"): read the fragments of all k-steps of a stage at once, double-buffered per
// stage, so a stage costs one LDS round trip instead of one per k-step.  For small wave tiles,
// whose k-steps hold too few MFMAs to cover the LDS latency.
//
// KG ("k-groups"): KG sets of WX x WY waves work on the same output tile, each set on its own
// share of the workgroup's reduction range with its own loaders and LDS buffers; their
// accumulators are summed through LDS before the epilogue.  For layers with few output tiles and
// a long reduction: KG times the loads in flight and KG waves per SIMD without device atomics.
template <int BX_, int BY_, int BKB_, int WX_, int WY_, bool FF_ = false, int KG_ = 1>
struct Tile {
  static constexpr int BX = BX_, BY = BY_, BKB = BKB_, WX = WX_, WY = WY_, KG = KG_;
  static constexpr bool FF = FF_;
  static constexpr int NTG = WX * WY * 64;       // threads of one k-group
  static constexpr int NT = NTG * KG;
  static constexpr int TX = BX / WX / 32, TY = BY / WY / 32;
  static constexpr int CPR = BKB / 16;           // 16-byte chunks per LDS row
  static constexpr int XBYTES = BX * BKB, YBYTES = BY * BKB;
  static constexpr int STAGE = XBYTES + YBYTES;
  static constexpr int LDS_TILES = 2 * STAGE * KG;
  // accumulators and weight sums of the k-groups other than the first, handed over through LDS
  static constexpr int XCHG = (KG - 1) * (BX * BY * 4 + (NTG / 64) * (TX + TY) * 256);
  static_assert(BX % (WX * 32) == 0 && BY % (WY * 32) == 0, "wave tile is a multiple of 32x32");
  static_assert(KG >= 1 && NT <= 1024, "at most 16 waves per workgroup");
};

// Workgroup id -> (tile, k-split).  Workgroups are dealt round-robin to the 8 XCDs, each with
// its own L2: ids congruent mod 8 share an XCD, so they are given consecutive logical ids, and
// logical ids walk the tile grid in panels `ph` X-tiles tall so that an XCD's working set is a
// compact patch of the grid.  The k-splits of one tile are adjacent logical ids.
struct GridMap {
  int gx, gy, ph, splits, total;  // total = gx * gy * splits
  // dividers by splits, by ph * gy (tiles per panel), by ph and by the height of the last panel: the walk costs a
  // few multiplies instead of three integer divisions at the head of every workgroup
  FastDiv by_splits, by_panel, by_ph, by_last;
  __host__ static GridMap make(int gx, int gy, int ph, int splits) {
    GridMap m;
    m.gx = gx;
    m.gy = gy;
    m.ph = ph < 1 ? 1 : (ph > gx ? gx : ph);
    m.splits = splits < 1 ? 1 : splits;
    m.total = gx * gy * m.splits;
    m.by_splits = FastDiv::make(m.splits);
    m.by_panel = FastDiv::make(m.ph * gy);
    m.by_ph = FastDiv::make(m.ph);
    m.by_last = FastDiv::make(gx % m.ph ? gx % m.ph : m.ph);
    return m;
  }
  __device__ __forceinline__ void locate(int bid, int &bx, int &by, int &split) const {
    constexpr int NXCD = 8;
    int per = total / NXCD, rem = total % NXCD;
    int xcd = bid % NXCD, idx = bid / NXCD;
    int logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
    split = 0;
    if (splits > 1) {
      int q;
      by_splits.divmod(logical, q, split);
      logical = q;
    }
    const int panel = by_panel.div(logical), within = logical - panel * (ph * gy);
    int rows = gx - panel * ph;
    const bool full = rows >= ph;
    rows = full ? ph : rows;
    FastDiv r;
    r.mul = full ? by_ph.mul : by_last.mul;
    r.shift = full ? by_ph.shift : by_last.shift;
    r.d = rows;
    int col;
    r.divmod(within, by, col);
    bx = panel * ph + col;
  }
};

enum { WS_NONE = 0, WS_X = 1, WS_Y = 2, WS_Y_GIVEN = 3, WS_Y_SPLIT = 4 };  // weight sums: none, summed in the kernel (X / Y rows), read from memory, summed in the kernel one Y block per wave

// The kernel.  XL / YL stage the operand tiles, Epi writes the accumulators.
// WS selects which operand is the s8 weight whose per-row byte sums are accumulated on the side
// (v_dot4 against 0x01010101): the u8 operand is staged as (u8 ^ 0x80) = u8 - 128 reinterpreted
// as s8, because the MFMA int8 path multiplies signed by signed, and the epilogue adds back
// 128 * sum_k w[k].  With k-splits each workgroup adds the correction of its own k-range.
//
// Schedule of one pipeline stage (KK = BKB / 32 MFMA k-steps, fragments double-buffered in
// registers):   ds_write stage+1 | global_load stage+2 | for kk: ds_read frags(kk+1), MFMA(kk) |
// before the last k-step: barrier, ds_read frags(0) of the next stage, then the last MFMAs --
// so LDS latency and the barrier skew are covered by MFMA work of the same wave.
template <class Op, class T, class XL, class YL, class Epi, int WS>
__global__ __launch_bounds__(T::NT) void mma_kernel(typename XL::Params xp, typename YL::Params yp,
                                                    typename Epi::Params ep, int nk_total, GridMap gm) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & 63;
  // k-group and wave inside it, as scalars: every branch below that depends on them is uniform
  const int wave_wg = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int grp = T::KG > 1 ? wave_wg / (T::WX * T::WY) : 0;
  const int wave = wave_wg - grp * (T::WX * T::WY);
  const int t = wave * 64 + lane;  // thread id inside the k-group
  const int wx = wave % T::WX, wy = wave / T::WX;
  const int l32 = lane & 31, half = lane >> 5;
  constexpr int KK = T::BKB / 32;
  static_assert(KK % 2 == 0, "fragment double buffering needs an even number of k-steps");

  int bx, by, split;
  gm.locate(blockIdx.x, bx, by, split);
  const int x0 = bx * T::BX, y0 = by * T::BY;
  // this workgroup's stages [kb0, ke0), this k-group's share of them [kb, ke)
  const int kb0 = (int)((long)nk_total * split / gm.splits), ke0 = (int)((long)nk_total * (split + 1) / gm.splits);
  const int kb = kb0 + (ke0 - kb0) * grp / T::KG, ke = kb0 + (ke0 - kb0) * (grp + 1) / T::KG;
  char *const tiles = lds + grp * (2 * T::STAGE);  // this k-group's LDS double buffer

  XL xl;
  YL yl;
  char *aux = lds + T::LDS_TILES;  // loader-private LDS (tap tables)
  xl.init(xp, x0, t, aux);
  yl.init(yp, y0, t, aux);

  typename Op::acc_t acc[T::TX][T::TY];
#pragma unroll
  for (int i = 0; i < T::TX; ++i)
#pragma unroll
    for (int j = 0; j < T::TY; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  int wsx[T::TX], wsy[T::TY];
#pragma unroll
  for (int i = 0; i < T::TX; ++i) wsx[i] = 0;
#pragma unroll
  for (int j = 0; j < T::TY; ++j) wsy[j] = 0;

  // per-lane LDS read offsets (row part); the swizzle only depends on row % 16 and every
  // 32-row block starts at a multiple of 32, so one mask serves all blocks of a lane
  const int xrow = wx * (T::TX * 32) + l32, yrow = wy * (T::TY * 32) + l32;
  const int xsw = swz<T::BKB>(xrow), ysw = swz<T::BKB>(yrow);
  const int xbase = xrow * T::BKB, ybase = T::XBYTES + yrow * T::BKB;

  constexpr int NSLOT = T::FF ? 2 * KK : 2;  // fragment register sets
  v4i xf[NSLOT][T::TX], yf[NSLOT][T::TY];
  auto load_frags = [&](const char *stage, int kk, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < T::TX; ++i)
      xf[slot][i] = *reinterpret_cast<const v4i *>(stage + xbase + i * 32 * T::BKB + (((2 * kk + half) ^ xsw) << 4));
#pragma unroll
    for (int j = 0; j < T::TY; ++j)
      yf[slot][j] = *reinterpret_cast<const v4i *>(stage + ybase + j * 32 * T::BKB + (((2 * kk + half) ^ ysw) << 4));
  };
  auto mma_step = [&](int slot) __attribute__((always_inline)) {
    if constexpr (WS == WS_X) {
#pragma unroll
      for (int i = 0; i < T::TX; ++i)
#pragma unroll
        for (int d = 0; d < 4; ++d) wsx[i] = __builtin_amdgcn_sdot4(xf[slot][i][d], 0x01010101, wsx[i], false);
    }
    if constexpr (WS == WS_Y) {
#pragma unroll
      for (int j = 0; j < T::TY; ++j)
#pragma unroll
        for (int d = 0; d < 4; ++d) wsy[j] = __builtin_amdgcn_sdot4(yf[slot][j][d], 0x01010101, wsy[j], false);
    }
#pragma unroll
    for (int i = 0; i < T::TX; ++i)
#pragma unroll
      for (int j = 0; j < T::TY; ++j) acc[i][j] = Op::mma(xf[slot][i], yf[slot][j], acc[i][j]);
  };

  // One pipeline stage.  U is the register slot that holds stage kt+1 (stages rotate through PF
  // slots, so PF stages of global loads are in flight).  NEXT: stage kt+1 exists (write it to
  // LDS, and after the barrier pre-load its first fragments); NEXTPF: stage kt+1+PF exists (fetch
  // it into the slot just freed).
  constexpr int PF = XL::kPF;
  static_assert(XL::kPF == YL::kPF, "both operands use the same prefetch depth");
  auto stage = [&](int kt, int par, auto slot, auto fset, bool next, bool nextpf) __attribute__((always_inline)) {
    constexpr int U = decltype(slot)::value;
    constexpr int FS = decltype(fset)::value;  // FF: fragment set that holds stage kt
    char *cur = tiles + par * T::STAGE;
    char *nxt = tiles + (par ^ 1) * T::STAGE;
    if (next) {
      xl.template commit<U>(nxt);
      yl.template commit<U>(nxt + T::XBYTES);
    }
    if (nextpf) {
      xl.template fetch<U>(kt + 1 + PF);
      yl.template fetch<U>(kt + 1 + PF);
    }
    if constexpr (T::FF) {
      // all fragments of `cur` were requested one stage ago; after the barrier (which also
      // waits for them) request all of `nxt`, then run the whole stage's MFMAs under those reads
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
      if (next) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) load_frags(nxt, kk, (FS ^ 1) * KK + kk);
      }
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) mma_step(FS * KK + kk);
    } else {
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        if (kk + 1 < KK) {
          load_frags(cur, kk + 1, (kk + 1) & 1);
          mma_step(kk & 1);
        } else {
          __builtin_amdgcn_sched_barrier(0);
          __syncthreads();  // everyone has read `cur` and written `nxt`
          if (next) load_frags(nxt, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          mma_step(kk & 1);
        }
      }
    }
  };
  // stage kt with the slot rotation resolved at compile time for PF consecutive stages
  auto stages_pf = [&](int kt, int par, auto steady) __attribute__((always_inline)) {
    auto one = [&](auto u) __attribute__((always_inline)) {
      constexpr int UU = decltype(u)::value;
      const int k = kt + UU;
      if constexpr (decltype(steady)::value) {
        stage(k, (par + UU) & 1, std::integral_constant<int, (UU + 1) % PF>{}, std::integral_constant<int, UU & 1>{}, true,
              true);
      } else {
        if (k < ke)
          stage(k, (par + UU) & 1, std::integral_constant<int, (UU + 1) % PF>{}, std::integral_constant<int, UU & 1>{},
                k + 1 < ke, k + 1 + PF < ke);
      }
    };
    one(std::integral_constant<int, 0>{});
    if constexpr (PF > 1) one(std::integral_constant<int, 1>{});
    if constexpr (PF > 2) one(std::integral_constant<int, 2>{});
    if constexpr (PF > 3) one(std::integral_constant<int, 3>{});
  };
  static_assert(PF >= 1 && PF <= 4, "prefetch depth 1..4");
  static_assert(!T::FF || PF % 2 == 0, "full-fragment mode alternates two fragment sets: even prefetch depth");

  if (XL::kNeedsSync || YL::kNeedsSync) __syncthreads();  // tap tables visible
  if (kb < ke) {
    // prologue: PF stages in flight, the first one staged into LDS
    xl.template fetch<0>(kb);
    yl.template fetch<0>(kb);
    if constexpr (PF > 1) {
      if (kb + 1 < ke) { xl.template fetch<1 % PF>(kb + 1); yl.template fetch<1 % PF>(kb + 1); }
    }
    if constexpr (PF > 2) {
      if (kb + 2 < ke) { xl.template fetch<2 % PF>(kb + 2); yl.template fetch<2 % PF>(kb + 2); }
    }
    if constexpr (PF > 3) {
      if (kb + 3 < ke) { xl.template fetch<3 % PF>(kb + 3); yl.template fetch<3 % PF>(kb + 3); }
    }
    xl.template commit<0>(tiles);
    yl.template commit<0>(tiles + T::XBYTES);
    if (kb + PF < ke) {
      xl.template fetch<0>(kb + PF);
      yl.template fetch<0>(kb + PF);
    }
    __syncthreads();
    if constexpr (T::FF) {
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) load_frags(tiles, kk, kk);
    } else {
      load_frags(tiles, 0, 0);
    }
    int kt = kb, par = 0;
    // steady state: every stage of the group has a successor and a stage PF+1 ahead to fetch
    for (; kt + 2 * PF < ke; kt += PF, par = (par + PF) & 1) stages_pf(kt, par, std::true_type{});
    for (; kt < ke; kt += PF, par = (par + PF) & 1) stages_pf(kt, par, std::false_type{});
  }

  // the two 32-lane halves hold the sums of the two 16-byte k-chunks of every MFMA step
  if constexpr (WS == WS_X) {
#pragma unroll
    for (int i = 0; i < T::TX; ++i) wsx[i] += __shfl_xor(wsx[i], 32);
  }
  if constexpr (WS == WS_Y) {
#pragma unroll
    for (int j = 0; j < T::TY; ++j) wsy[j] += __shfl_xor(wsy[j], 32);
  }

  if constexpr (T::KG > 1) {
    // Every k-group must arrive at the same number of workgroup barriers: one in the prologue
    // and one per stage, for the group with the most stages.
    const int mine = ke - kb, most = (ke0 - kb0 + T::KG - 1) / T::KG;
    for (int i = mine > 0 ? 1 + mine : 0; i < 1 + most; ++i) __syncthreads();
    // Hand the partial sums to the first k-group.  The exchange area lies behind the LDS the
    // epilogue uses, so a wave that starts its epilogue early cannot overwrite it.
    constexpr int NW = T::NTG / 64, NB = T::TX * T::TY;
    char *xch = lds + Epi::template lds_bytes<T>();
    int *xws = reinterpret_cast<int *>(xch + (T::KG - 1) * (T::BX * T::BY * 4));
    if (grp > 0) {
      char *mine_acc = xch + ((grp - 1) * NW + wave) * (NB * 4096);
      int *mine_ws = xws + ((grp - 1) * NW + wave) * ((T::TX + T::TY) * 64);
#pragma unroll
      for (int i = 0; i < T::TX; ++i)
#pragma unroll
        for (int j = 0; j < T::TY; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *reinterpret_cast<typename Op::out4_t *>(mine_acc + (((i * T::TY + j) * 4 + q) * 64 + lane) * 16) =
                typename Op::out4_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
#pragma unroll
      for (int i = 0; i < T::TX; ++i) mine_ws[i * 64 + lane] = wsx[i];
#pragma unroll
      for (int j = 0; j < T::TY; ++j) mine_ws[(T::TX + j) * 64 + lane] = wsy[j];
    }
    __syncthreads();
    if (grp > 0) return;
#pragma unroll
    for (int g = 1; g < T::KG; ++g) {
      const char *its_acc = xch + ((g - 1) * NW + wave) * (NB * 4096);
      const int *its_ws = xws + ((g - 1) * NW + wave) * ((T::TX + T::TY) * 64);
#pragma unroll
      for (int i = 0; i < T::TX; ++i)
#pragma unroll
        for (int j = 0; j < T::TY; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const auto v = *reinterpret_cast<const typename Op::out4_t *>(its_acc + (((i * T::TY + j) * 4 + q) * 64 + lane) * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] += v[e];
          }
#pragma unroll
      for (int i = 0; i < T::TX; ++i) wsx[i] += its_ws[i * 64 + lane];
#pragma unroll
      for (int j = 0; j < T::TY; ++j) wsy[j] += its_ws[(T::TX + j) * 64 + lane];
    }
  }

  // the last barrier of the K loop came after every LDS read: the tiles are free for the epilogue
  if constexpr (Epi::kSplitPlanes)  // every k-split writes a plane of its own: the last argument is the split
    Epi::template store<T>(ep, acc, wsx, wsy, x0 + wx * (T::TX * 32), y0 + wy * (T::TY * 32), lane, wave, lds, split);
  else
    Epi::template store<T>(ep, acc, wsx, wsy, x0 + wx * (T::TX * 32), y0 + wy * (T::TY * 32), lane, wave, lds,
                           gm.splits > 1);
}

// zero fill for outputs accumulated with atomics (k-splits): 16 bytes per thread
static __global__ __launch_bounds__(256) void zero_fill(v4i *dst, size_t n16) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) dst[i] = v4i{0, 0, 0, 0};
}

}  // namespace unit
