// GEMM kernel whose operand tiles go global -> LDS directly (global_load_lds_dwordx4, no VGPR
// round trip) through a ring of NSTAGE LDS buffers, so NSTAGE-1 stages of loads are in flight
// while one is consumed.  Both operands must be K-contiguous rows (A (M, K) and W (N, K)) and the
// reduction a whole number of stages; everything else uses mma_kernel.
//
// A wave-level direct load writes 64 lanes x 16 bytes = 1 KiB of consecutive LDS, so lane i
// fetches the global chunk that belongs at LDS position i of that KiB: LDS rows keep the same
// XOR-swizzled [row][BKB] layout the MFMA fragment reads of mma_kernel use.  The u8 operand
// cannot be shifted to s8 on the way, so it is shifted after the fragment read (4 v_xor per
// fragment).
#pragma once
#include "mma_core.hpp"
#include "trace.hpp"

namespace unit {

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

// s_waitcnt vmcnt(n) only (expcnt / lgkmcnt fields left at "no wait"), gfx9 encoding
#define UNIT_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

struct DmaParams {
  const char *x;  // X rows (first MFMA operand), K-contiguous
  const char *y;  // Y rows
  int xrows, yrows;
  int ld;         // bytes per row (both operands)
  const int *ysum;  // WS_Y_GIVEN: sum of each Y row's bytes (the int8 weight sums), computed once per weight
  int ldy = 0;      // YT: bytes per k row of the (K, yrows) Y operand
};

typedef short v4s __attribute__((ext_vector_type(4)));

// One wave-level direct load (64 lanes x 16 B -> 1 KiB of LDS at lds_addr) written out as instructions.  A direct
// load that the compiler knows of costs twice: it counts the load on the LDS counter as well, after which every wait
// for a fragment read becomes a wait for all of them (lgkmcnt(0) at the head of every k-step), and it makes the
// transposing LDS read wait for all direct loads in flight (it cannot tell which LDS bytes a load fills), which
// undoes the ring.  Loads issued this way are invisible to it, so the kernel's own vmcnt waits order them alone.
// m0 is a register the compiler reserves: it never keeps a value in it across statements (it writes m0 right before
// each instruction of its own that reads it), so the statement may overwrite it; naming it as a clobber is rejected
// ("clobber list contains reserved registers").
__device__ __forceinline__ void direct_load_16(const void *src, u32 lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(src)
               : "memory");
}
// The same with the address as a wave-uniform base (SGPR pair) plus a 32-bit lane offset, and the LDS position in an
// SGPR: no vector instruction is spent on addresses, and no vector -> scalar hand-over sits in front of the load.
// (Cache-policy bits on these loads were measured at 4096^3: sc0 / sc1 within noise, nt 6-15 % slower.)
__device__ __forceinline__ void direct_load_16s(const void *sbase, u32 voff, u32 lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(sbase)
               : "memory");
}

// YT (16-bit operands only): Y is given reduction-major, (K, yrows) with yrows contiguous -- the fp16 GEMM's b as the
// reference has it.  Its tile lands in LDS as it lies in memory, [k][BY / 8 chunks of 8 columns], and the MFMA
// fragments (8 consecutive k of one column per lane) come out of it with the LDS transposing read
// (ds_read_b64_tr_b16): within 16 lanes, source lanes 4r .. 4r+3 hand in 16 consecutive columns of k row r and lane
// i receives column i of the four rows.  Two such reads make one fragment.  The chunk position inside a k row is
// XORed with 4 * (k % 4), so that the four rows of a read fall into different bank groups (rows are 256 or 512 B).
template <class Op, class T, int NSTAGE, class Epi, int WS, bool XOR_X, bool YT = false>
__global__ __launch_bounds__(T::NT) void mma_dma_kernel(DmaParams p, typename Epi::Params ep, int nk, GridMap gm
                                                        UNIT_TRACE(, unsigned long long *trace_buf)) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  // timeline: 0 entry, 1 ring issued, 2 stage 0 landed (after the barrier), 3 last MFMA done, 4 stores issued,
  // 5 stores acknowledged; 8 loop ticks, 9 ticks waiting for direct loads, 10 ticks in lgkmcnt + barrier, 11 entry -> loop
  UNIT_TRACE(WaveTrace tr; tr.mark(0); const unsigned long long tk_entry = WaveTrace::ticks();
             unsigned long long tk_a = 0, tk_b = 0, tk_c = 0, tk_vm = 0, tk_bar = 0;)
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // wave-uniform: LDS positions of the direct loads stay scalar
  const u32 ring_addr = (u32)(uintptr_t)(lptr_t)lds;
  const int wx = wave % T::WX, wy = wave / T::WX;
  const int l32 = lane & 31, half = lane >> 5;
  constexpr int KK = T::BKB / 32, CPR = T::CPR, NW = T::NT / 64;
  constexpr int RPL = 64 / CPR;                  // rows per wave-level load (1 KiB)
  constexpr int XL = T::BX / RPL / NW;           // loads per wave per stage, X tile
  constexpr int YL = T::BY / RPL / NW;
  static_assert(T::BX % (RPL * NW) == 0 && T::BY % (RPL * NW) == 0, "tile rows split evenly over the waves");
  static_assert(KK % 2 == 0, "fragment double buffering needs an even number of k-steps");
  constexpr int LPS = XL + YL;                   // loads per wave per stage
  constexpr int CPRY = T::BY / 8, RPLY = 64 / CPRY;  // YT: chunks per k row, k rows per wave-level load
  static_assert(!YT || (CPRY >= 16 && CPRY <= 64 && (T::BKB / 2) % (RPLY * NW) == 0 && YL == T::BKB / 2 / RPLY / NW &&
                        WS == WS_NONE && !XOR_X), "transposed-Y tile shape");
  // WS_Y_SPLIT: the WX waves that read the same Y fragments (same wy) share the weight sums: wave wx reads the Y
  // blocks of its tile rotated by wx, so the block it sums is always its fragment 0 (four v_dot4 per k-step and wave
  // instead of 4 * TY), and the waves exchange their sums through LDS after the loop.
  constexpr bool SPLIT = WS == WS_Y_SPLIT;
  static_assert(!SPLIT || (T::TY == T::WX && (T::TY & (T::TY - 1)) == 0 && T::TX * T::TY >= 6 && !YT),
                "split weight sums: one Y block per wave of a row of waves");

  int bx, by, split;
  gm.locate(blockIdx.x, bx, by, split);
  const int x0 = bx * T::BX, y0 = by * T::BY;
  const size_t ystep = YT ? (size_t)(T::BKB / 2) * p.ldy : (size_t)T::BKB;  // Y bytes from one stage to the next
  if (gm.splits > 1) {  // this workgroup's share of the stages: [first, first + nk)
    const int per = nk / gm.splits, rem = nk % gm.splits;
    const int first = split * per + (split < rem ? split : rem);
    nk = per + (split < rem ? 1 : 0);
    p.x += (size_t)first * T::BKB;
    p.y += (size_t)first * ystep;
  }

  // per-lane source offsets: lane -> (row, slot) of its KiB, chunk = slot ^ swizzle(row)
  u32 xoff[XL], yoff[YL];
  const int lrow = lane / CPR, slot = lane % CPR;
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int row = (wave * XL + i) * RPL + lrow;
    int g = x0 + row;
    g = g < p.xrows ? g : p.xrows - 1;
    xoff[i] = (u32)g * (u32)p.ld + ((slot ^ swz<T::BKB>(row)) << 4);
  }
#pragma unroll
  for (int i = 0; i < YL; ++i) {
    if constexpr (YT) {
      const int krow = (wave * YL + i) * RPLY + lane / CPRY;
      int c = y0 / 8 + ((lane % CPRY) ^ (4 * (krow & 3)));
      c = c < p.yrows / 8 ? c : p.yrows / 8 - 1;
      yoff[i] = (u32)krow * (u32)p.ldy + ((u32)c << 4);
    } else {
      const int row = (wave * YL + i) * RPL + lrow;
      int g = y0 + row;
      g = g < p.yrows ? g : p.yrows - 1;
      yoff[i] = (u32)g * (u32)p.ld + ((slot ^ swz<T::BKB>(row)) << 4);
    }
  }

  // load i of stage kt's LPS loads of this wave, into ring buffer `slot`
  auto issue_one = [&](int kt, int slot, int i) {
    const u32 buf = ring_addr + (u32)(slot * T::STAGE);
    if (i < XL)
      direct_load_16s(p.x + (size_t)kt * T::BKB, xoff[i], buf + (wave * XL + i) * 1024);
    else
      direct_load_16s(p.y + (size_t)kt * ystep, yoff[i - XL], buf + T::XBYTES + (wave * YL + (i - XL)) * 1024);
  };
  auto issue = [&](int kt) {
#pragma unroll
    for (int i = 0; i < LPS; ++i) issue_one(kt, kt % NSTAGE, i);
  };

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

  const int xrow = wx * (T::TX * 32) + l32, yrow = wy * (T::TY * 32) + l32;
  const int xsw = swz<T::BKB>(xrow), ysw = swz<T::BKB>(yrow);  // the swizzle repeats every 16 rows
  const int xbase = xrow * T::BKB, ybase = T::XBYTES + yrow * T::BKB;
  const int yrot = SPLIT ? wx : 0;
  int yblk[T::TY];  // fragment j of this wave is Y block (j + yrot) % TY of the wave tile
#pragma unroll
  for (int j = 0; j < T::TY; ++j) yblk[j] = ybase + ((j + yrot) % T::TY) * 32 * T::BKB;

  // YT: byte offset, inside the Y tile, of what this lane hands to the transposing reads of fragment j at k-step 0,
  // read 0: k row 8 * half + (lane % 16) / 4, columns 32 j + 16 * ((lane / 16) % 2) + 4 * (lane % 4) .. + 3
  int ytr[T::TY];
  if constexpr (YT) {
    const int jrow = (lane & 15) >> 2, q = lane & 3, g16 = (lane >> 4) & 1;
#pragma unroll
    for (int j = 0; j < T::TY; ++j) {
      const int c = wy * (T::TY * 4) + j * 4 + 2 * g16 + (q >> 1);
      ytr[j] = (8 * half + jrow) * (T::BY * 2) + ((c ^ (4 * jrow)) << 4) + (q & 1) * 8;
    }
  }

  v4i xf[2][T::TX], yf[2][T::TY];
  // fragment i of the step's read list: X0, Y0..Y(TY-1), X1..X(TX-1) -- the first MFMA needs
  // only the first two
  auto load_one = [&](const char *stage, int kk, int s, int idx) {
    const int cx = ((2 * kk + half) ^ xsw) << 4, cy = ((2 * kk + half) ^ ysw) << 4;
    if (idx == 0)
      xf[s][0] = *reinterpret_cast<const v4i *>(stage + xbase + cx);
    else if (idx <= T::TY) {
      if constexpr (YT) {
        typedef __attribute__((address_space(3))) v4s *trptr_t;
        typedef short v8s __attribute__((ext_vector_type(8)));
        const char *src = stage + T::XBYTES + ytr[idx - 1] + kk * 16 * (T::BY * 2);
        const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((trptr_t)(src));
        const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((trptr_t)(src + 4 * (T::BY * 2)));
        yf[s][idx - 1] = __builtin_bit_cast(v4i, (v8s)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      } else {
        yf[s][idx - 1] = *reinterpret_cast<const v4i *>(stage + (SPLIT ? yblk[idx - 1] : ybase + (idx - 1) * 32 * T::BKB) + cy);
      }
    }
    else
      xf[s][idx - T::TY] = *reinterpret_cast<const v4i *>(stage + xbase + (idx - T::TY) * 32 * T::BKB + cx);
  };
  auto load_frags = [&](const char *stage, int kk, int s) {
#pragma unroll
    for (int i = 0; i < T::TX + T::TY; ++i) load_one(stage, kk, s, i);
  };
  // One k-step with a fixed instruction order: every MFMA is followed by one slice of the
  // step's other work (a fragment read for the next step, a direct load for a later stage, the
  // u8 -> s8 shift of the next X fragment, one weight-sum dot) and a scheduling fence, because
  // with one wave per SIMD only instructions placed between two MFMAs overlap with them.
  //   s: fragment slot consumed;  rd_stage/rd_kk: where the next step's fragments come from
  //   (nullptr: none);  issue_kt >= 0: stage to fetch with direct loads.
  auto step = [&](int s, const char *rd_stage, int rd_kk, int issue_kt, int issue_slot, auto has_read, auto has_issue) {
    constexpr int NM = T::TX * T::TY, NF = T::TX + T::TY;
    if constexpr (XOR_X) xf[s][0] ^= (int)0x80808080;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      const int i = m / T::TY, j = m % T::TY;
      acc[i][j] = Op::mma(xf[s][i], yf[s][j], acc[i][j]);
      if constexpr (decltype(has_read)::value) {
        if (m < NF) load_one(rd_stage, rd_kk, s ^ 1, m);
      }
      if constexpr (decltype(has_issue)::value) {
        if (m >= NM - LPS) issue_one(issue_kt, issue_slot, m - (NM - LPS));
      }
      if constexpr (XOR_X) {
        if (j == T::TY - 1 && i + 1 < T::TX) xf[s][i + 1] ^= (int)0x80808080;
      }
      if constexpr (SPLIT) {
        if (m >= 2 && m < 6) wsy[0] = __builtin_amdgcn_sdot4(yf[s][0][m - 2], 0x01010101, wsy[0], false);
      }
      if constexpr (WS == WS_Y) {
        // TY fragments x 4 dwords spread over the step's MFMAs, DPM dots after each
        constexpr int DPM = (4 * T::TY + NM - 1) / NM;
#pragma unroll
        for (int d = 0; d < DPM; ++d) {
          const int w = m * DPM + d;
          if (w < 4 * T::TY) wsy[w / 4] = __builtin_amdgcn_sdot4(yf[s][w / 4][w % 4], 0x01010101, wsy[w / 4], false);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  static_assert(T::TX * T::TY >= LPS && T::TX * T::TY >= T::TX + T::TY,
                "not enough MFMAs per k-step to carry the step's other work");

  // One stage.  ISSUE: stage kt + NSTAGE exists and is fetched into the buffer this stage
  // frees; STEADY: NSTAGE-1 younger stages are in flight when the barrier is reached (else
  // wait for everything); NEXT: stage kt + 1 exists.
  // slot: the ring buffer of stage kt (kt % NSTAGE; a constant in the unrolled steady-state loop, so that every LDS
  // address of a stage is a register plus an immediate)
  auto stage = [&](int kt, int slot, auto issue_next, auto steady, auto next) {
    const char *cur = lds + slot * T::STAGE;
    const int slot_next = slot + 1 == NSTAGE ? 0 : slot + 1;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) {
        step(kk & 1, cur, kk + 1, -1, 0, std::true_type{}, std::false_type{});
      } else {
        // stage kt+1 must have landed; stages kt+2 .. kt+NSTAGE-1 may stay in flight
        UNIT_TRACE(tk_bar += tk_c - tk_b; tk_a = WaveTrace::ticks(); __builtin_amdgcn_sched_barrier(0);)
        if constexpr (decltype(steady)::value)
          UNIT_WAIT_VMCNT((NSTAGE - 2) * LPS);
        else
          UNIT_WAIT_VMCNT(0);
        UNIT_TRACE(__builtin_amdgcn_sched_barrier(0); tk_b = WaveTrace::ticks(); __builtin_amdgcn_sched_barrier(0);)
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's reads of `cur` are done
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        UNIT_TRACE(tk_vm += tk_b - tk_a; tk_c = WaveTrace::ticks(); __builtin_amdgcn_sched_barrier(0);)
        // every wave has read stage kt: its buffer takes stage kt + NSTAGE
        step(kk & 1, lds + slot_next * T::STAGE, 0, kt + NSTAGE, slot, next, issue_next);
      }
    }
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;

  // prologue: fill the ring
#pragma unroll
  for (int s = 0; s < NSTAGE; ++s)
    if (s < nk) issue(s);
  UNIT_TRACE(tr.mark(1);)
  // stage 0 landed?  (the NSTAGE-1 younger stages may still be in flight)
  if (nk >= NSTAGE)
    UNIT_WAIT_VMCNT((NSTAGE - 1) * LPS);
  else
    UNIT_WAIT_VMCNT(0);
  __builtin_amdgcn_s_barrier();
  UNIT_TRACE(tr.mark(2); const unsigned long long tk_loop = WaveTrace::ticks(); tk_b = tk_c = tk_loop;)
  load_frags(lds, 0, 0);

  int kt = 0;
  for (; kt + 2 * NSTAGE <= nk; kt += NSTAGE) {  // steady state, unrolled by the ring: kt % NSTAGE == 0 here
#pragma unroll
    for (int s = 0; s < NSTAGE; ++s) stage(kt + s, s, yes{}, yes{}, yes{});
  }
  for (; kt + NSTAGE < nk; ++kt) stage(kt, kt % NSTAGE, yes{}, yes{}, yes{});
  for (; kt + 1 < nk; ++kt) stage(kt, kt % NSTAGE, no{}, no{}, yes{});
  if (kt < nk) stage(kt, kt % NSTAGE, no{}, no{}, no{});
  UNIT_TRACE(asm volatile("s_nop 0" ::"v"(acc[T::TX - 1][T::TY - 1][15]));  // the last MFMA has written its result
             tr.mark(3); tr.w[8] = WaveTrace::ticks() - tk_loop; tr.w[9] = tk_vm; tr.w[10] = tk_bar;
             tr.w[11] = tk_loop - tk_entry;)

  if constexpr (WS == WS_Y) {
#pragma unroll
    for (int j = 0; j < T::TY; ++j) wsy[j] += __shfl_xor(wsy[j], 32);
  }
  if constexpr (SPLIT) {
    // The ring buffer that the last stage does not use is free once its barrier is passed: the waves leave the sums
    // of their blocks there, [wy][block][32 rows], and pick up all TY blocks of their row of waves.
    int *sums = reinterpret_cast<int *>(lds + ((nk + NSTAGE - 2) % NSTAGE) * T::STAGE);
    const int part = wsy[0] + __shfl_xor(wsy[0], 32);
    if (half == 0) sums[(wy * T::TY + yrot) * 32 + l32] = part;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < T::TY; ++j) wsy[j] = sums[(wy * T::TY + ((j + yrot) % T::TY)) * 32 + l32];
  }
  if constexpr (WS == WS_Y_GIVEN) {
#pragma unroll
    for (int j = 0; j < T::TY; ++j) {
      const int n = y0 + wy * (T::TY * 32) + j * 32 + l32;
      wsy[j] = n < p.yrows && split == 0 ? p.ysum[n] : 0;  // one k-split adds the whole row's sum
    }
  }
  if constexpr (Epi::kSplitPlanes)  // every k-split writes a plane of its own: the last argument is the split
    Epi::template store<T>(ep, acc, wsx, wsy, x0 + wx * (T::TX * 32), y0 + wy * (T::TY * 32), lane, wave, lds, split);
  else
    Epi::template store<T>(ep, acc, wsx, wsy, x0 + wx * (T::TX * 32), y0 + wy * (T::TY * 32), lane, wave, lds,
                           gm.splits > 1, yrot);
  UNIT_TRACE(tr.mark(4); __builtin_amdgcn_s_waitcnt(0x0F70); tr.mark(5); tr.flush(trace_buf, blockIdx.x * NW + wave);)
}

}  // namespace unit

namespace unit {

// Hybrid of the two pipelines: the X operand (K-contiguous rows) goes global -> LDS directly
// through a two-buffer ring, the Y operand through a register loader (YRL: fetch to registers,
// commit to LDS), for operands that have to be transposed on the way (the fp16 GEMM's b (K, N)).
//
// Stage kt computes from buffer kt % 2.  Y(kt + 2) is fetched into registers at the start of stage
// kt and committed into the same buffer right after the barrier that ends the reads of stage kt;
// X(kt + 2) is issued there too.  vmcnt accounting: when the barrier of stage kt is reached the
// outstanding loads are X(kt + 1) (older) and the Y(kt + 2) fetches (younger, YRL::kLoads of them).
template <class Op, class T, class YRL, class Epi>
__global__ __launch_bounds__(T::NT) void mma_hybrid_kernel(DmaParams p, typename YRL::Params yp, typename Epi::Params ep,
                                                           int nk, GridMap gm) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int wx = wave % T::WX, wy = wave / T::WX;
  const int l32 = lane & 31, half = lane >> 5;
  constexpr int KK = T::BKB / 32, CPR = T::CPR, NW = T::NT / 64;
  constexpr int RPL = 64 / CPR;
  constexpr int XL = T::BX / RPL / NW;
  static_assert(T::BX % (RPL * NW) == 0 && KK % 2 == 0 && YRL::kPF == 1, "hybrid kernel shape");
  constexpr int NM = T::TX * T::TY, NF = T::TX + T::TY;
  static_assert(NM >= XL && NM >= NF, "not enough MFMAs per k-step to carry the step's other work");

  int bx, by, split;
  gm.locate(blockIdx.x, bx, by, split);
  const int x0 = bx * T::BX, y0 = by * T::BY;

  u32 xoff[XL];
  const int lrow = lane / CPR, slot = lane % CPR;
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int row = (wave * XL + i) * RPL + lrow;
    int g = x0 + row;
    g = g < p.xrows ? g : p.xrows - 1;
    xoff[i] = (u32)g * (u32)p.ld + ((slot ^ swz<T::BKB>(row)) << 4);
  }
  YRL yl;
  yl.init(yp, y0, t, nullptr);

  auto issue_one = [&](int kt, int i) {
    char *buf = lds + (kt & 1) * T::STAGE;
    const char *xs = p.x + (size_t)kt * T::BKB;
    __builtin_amdgcn_global_load_lds((gptr_t)(xs + xoff[i]), (lptr_t)(buf + (wave * XL + i) * 1024), 16, 0, 0);
  };

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

  const int xrow = wx * (T::TX * 32) + l32, yrow = wy * (T::TY * 32) + l32;
  const int xsw = swz<T::BKB>(xrow), ysw = swz<T::BKB>(yrow);
  const int xbase = xrow * T::BKB, ybase = T::XBYTES + yrow * T::BKB;

  v4i xf[2][T::TX], yf[2][T::TY];
  auto load_one = [&](const char *stage, int kk, int s, int idx) {
    const int cx = ((2 * kk + half) ^ xsw) << 4, cy = ((2 * kk + half) ^ ysw) << 4;
    if (idx == 0)
      xf[s][0] = *reinterpret_cast<const v4i *>(stage + xbase + cx);
    else if (idx <= T::TY)
      yf[s][idx - 1] = *reinterpret_cast<const v4i *>(stage + ybase + (idx - 1) * 32 * T::BKB + cy);
    else
      xf[s][idx - T::TY] = *reinterpret_cast<const v4i *>(stage + xbase + (idx - T::TY) * 32 * T::BKB + cx);
  };
  // one k-step: MFMAs with one slice of other work after each
  auto step = [&](int s, const char *rd_stage, int rd_kk, int issue_kt, auto has_read, auto has_issue) {
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      const int i = m / T::TY, j = m % T::TY;
      acc[i][j] = Op::mma(xf[s][i], yf[s][j], acc[i][j]);
      if constexpr (decltype(has_read)::value) {
        if (m < NF) load_one(rd_stage, rd_kk, s ^ 1, m);
      }
      if constexpr (decltype(has_issue)::value) {
        if (m >= NM - XL) issue_one(issue_kt, m - (NM - XL));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;

  // AHEAD: stage kt + 2 exists (fetched at the start, committed / issued after the barrier);
  // NEXT: stage kt + 1 exists
  auto stage = [&](int kt, auto ahead, auto next) {
    const char *cur = lds + (kt & 1) * T::STAGE;
    char *other = lds + ((kt + 1) & 1) * T::STAGE;
    if constexpr (decltype(ahead)::value) yl.template fetch<0>(kt + 2);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) {
        step(kk & 1, cur, kk + 1, -1, yes{}, no{});
      } else {
        // X(kt + 1) must have landed; the Y(kt + 2) fetches may stay in flight
        if constexpr (decltype(ahead)::value)
          UNIT_WAIT_VMCNT(YRL::kLoads);
        else
          UNIT_WAIT_VMCNT(0);
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's reads of `cur` are done
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (decltype(ahead)::value) yl.template commit<0>(const_cast<char *>(cur) + T::XBYTES);
        step(kk & 1, other, 0, kt + 2, next, ahead);
      }
    }
  };

  // prologue: X(0), X(1) by direct loads, Y(0), Y(1) through registers
#pragma unroll
  for (int s = 0; s < 2; ++s)
    if (s < nk) {
#pragma unroll
      for (int i = 0; i < XL; ++i) issue_one(s, i);
      yl.template fetch<0>(s);
      yl.template commit<0>(lds + s * T::STAGE + T::XBYTES);
    }
  UNIT_WAIT_VMCNT(0);
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < NF; ++i) load_one(lds, 0, 0, i);

  int kt = 0;
  for (; kt + 2 < nk; ++kt) stage(kt, yes{}, yes{});
  for (; kt + 1 < nk; ++kt) stage(kt, no{}, yes{});
  if (kt < nk) stage(kt, no{}, no{});

  Epi::template store<T>(ep, acc, wsx, wsy, x0 + wx * (T::TX * 32), y0 + wy * (T::TY * 32), lane, wave, lds, false);
}

}  // namespace unit
