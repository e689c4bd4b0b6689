// fp16 GEMM: c (M, N) = a (M, K) f16 . b (K, N) f16, fp32 accumulate on v_mfma_f32_32x32x16_f16.
// X operand = a (rows m, K-contiguous), Y operand = b (rows n, transposed while staging).
#include <mutex>

#include "epilogues.hpp"
#include "host.hpp"
#include "loaders.hpp"
#include "mma_dma.hpp"

namespace unit {
namespace {

// Prepared b: (N, K) rows, K-contiguous like a.  Both operands then go global -> LDS directly
// (no register round trip, no transposition), through a ring of NSTAGE LDS buffers; K a whole
// number of stages.
template <class T, int NSTAGE, bool OUT_F16>
int run_gemm_f16_bt_dma(const void *a, const void *bt, void *c, int M, int N, int K, hipStream_t s, int splits = 1) {
  using Epi = GemmEpilogue<OpF16, OUT_F16>;
  DmaParams p{static_cast<const char *>(a), static_cast<const char *>(bt), M, N, K * 2, nullptr};
  typename Epi::Params ep{c, M, N};
  const int nk = K * 2 / T::BKB, gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
  constexpr int lds = NSTAGE * T::STAGE;
  static_assert(lds <= kMaxLds, "ring does not fit the LDS");
  auto kern = mma_dma_kernel<OpF16, T, NSTAGE, Epi, WS_NONE, false>;
  static thread_local bool allowed = false;
  if (!allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "unit_gemm_f16_prepared: hipFuncSetAttribute: %s", hipGetErrorString(e));
    allowed = true;
  }
  splits = OUT_F16 || splits < 1 ? 1 : (splits > nk ? nk : splits);
  if (splits > 1) {  // the k-ranges add into c with atomics
    const size_t n16 = (size_t)M * N * 4 / 16;
    hipLaunchKernelGGL(zero_fill, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, s, static_cast<v4i *>(c), n16);
  }
  const GridMap gm = GridMap::make(gx, gy, gx < 4 ? gx : 4, splits);
  set_variant("f16gemmbt_dma_x%d_y%d_k%d_w%dx%d_r%d%s_s%d", T::BX, T::BY, T::BKB, T::WX, T::WY, NSTAGE, OUT_F16 ? "_h" : "",
              splits);
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(T::NT), lds, s, p, ep, nk, gm UNIT_TRACE(, trace_buffer()));
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "unit_gemm_f16_prepared: launch: %s", hipGetErrorString(e));
}

// b (K, N) as the reference gives it, both operands global -> LDS directly: b's tile lands as it lies in memory and
// the fragments come out of it with the LDS transposing read (K a whole number of stages, N a multiple of 8).
// splits > 1: k-ranges, added with atomics into the zero-filled c (Epi = GemmEpilogue, f32) or written as planes.
template <class T, int NSTAGE, class Epi>
int run_gemm_f16_dma_tr(const char *what, const char *tag, const void *a, const void *b, const typename Epi::Params &ep,
                        int M, int N, int K, int splits, void *zero, hipStream_t s) {
  DmaParams p{static_cast<const char *>(a), static_cast<const char *>(b), M, N, K * 2, nullptr, N * 2};
  const int nk = K * 2 / T::BKB, gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
  constexpr int lds = NSTAGE * T::STAGE;
  static_assert(lds <= kMaxLds, "ring does not fit the LDS");
  auto kern = mma_dma_kernel<OpF16, T, NSTAGE, Epi, WS_NONE, false, true>;
  static thread_local bool allowed = false;
  if (!allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
    allowed = true;
  }
  splits = splits < 1 ? 1 : (splits > nk ? nk : splits);
  if (splits > 1 && zero) {
    const size_t n16 = (size_t)M * N * 4 / 16;
    hipLaunchKernelGGL(zero_fill, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, s, static_cast<v4i *>(zero), n16);
  }
  const GridMap gm = GridMap::make(gx, gy, gx < 4 ? gx : 4, splits);
  set_variant("f16gemm_%s_x%d_y%d_k%d_w%dx%d_r%d_s%d", tag, T::BX, T::BY, T::BKB, T::WX, T::WY, NSTAGE, splits);
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(T::NT), lds, s, p, ep, nk, gm UNIT_TRACE(, trace_buffer()));
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
}

template <class T, int NSTAGE, bool OUT_F16>
int run_gemm_f16_dma_tr(const void *a, const void *b, void *c, int M, int N, int K, hipStream_t s, int splits = 1) {
  using Epi = GemmEpilogue<OpF16, OUT_F16>;
  typename Epi::Params ep{c, M, N};
  return run_gemm_f16_dma_tr<T, NSTAGE, Epi>("unit_gemm_f16", OUT_F16 ? "dmatr_h" : "dmatr", a, b, ep, M, N, K,
                                             OUT_F16 ? 1 : splits, c, s);
}

// b (K, N): a goes global -> LDS directly, b through the transposing register loader (K a whole number of stages)
template <class T, bool OUT_F16>
int run_gemm_f16_hybrid(const void *a, const void *b, void *c, int M, int N, int K, hipStream_t s) {
  using YL = KMajorF16Loader<T::BY, T::BKB, T::NT, 1, false>;
  using Epi = GemmEpilogue<OpF16, OUT_F16>;
  DmaParams p{static_cast<const char *>(a), nullptr, M, N, K * 2, nullptr};
  typename YL::Params yp{static_cast<const char *>(b), N, K, N + 4, 0, N * 2};
  typename Epi::Params ep{c, M, N};
  const int nk = K * 2 / T::BKB, gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
  constexpr int lds = 2 * T::STAGE;
  auto kern = mma_hybrid_kernel<OpF16, T, YL, Epi>;
  static thread_local bool allowed = false;
  if (!allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "unit_gemm_f16: hipFuncSetAttribute: %s", hipGetErrorString(e));
    allowed = true;
  }
  const GridMap gm = GridMap::make(gx, gy, gx < 4 ? gx : 4, 1);
  set_variant("f16gemm_hybrid_x%d_y%d_k%d_w%dx%d%s", T::BX, T::BY, T::BKB, T::WX, T::WY, OUT_F16 ? "_h" : "");
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(T::NT), lds, s, p, yp, ep, nk, gm);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "unit_gemm_f16: launch: %s", hipGetErrorString(e));
}

// the same operands through registers (any K that is a multiple of 8; small problems)
template <class T, bool OUT_F16>
int run_gemm_f16_bt(const void *a, const void *bt, void *c, int M, int N, int K, hipStream_t s) {
  using XL = RowMajorLoader<T::BX, T::BKB, T::NT, false>;
  using YL = RowMajorLoader<T::BY, T::BKB, T::NT, false>;
  using Epi = GemmEpilogue<OpF16, OUT_F16>;
  typename XL::Params xp{static_cast<const char *>(a), M, K * 2, K * 2};
  typename YL::Params yp{static_cast<const char *>(bt), N, K * 2, K * 2};
  typename Epi::Params ep{c, M, N};
  const int nk = ceil_div(K * 2, T::BKB), gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
  const int splits = OUT_F16 ? 1 : gemm_k_splits("UNIT_AMD_GEMM_F16_SPLITK", M, N, 2l * K, nk);
  set_variant("f16gemmbt_x%d_y%d_k%d_w%dx%d%s_s%d", T::BX, T::BY, T::BKB, T::WX, T::WY, OUT_F16 ? "_h" : "", splits);
  return launch_mma<OpF16, T, XL, YL, Epi, WS_NONE>(xp, yp, ep, nk, gx, gy, 4, splits, c, (size_t)M * N * 4, 0, s,
                                                    "unit_gemm_f16_prepared");
}

template <bool OUT_F16>
int gemm_f16_bt(const void *a, const void *bt, void *c, int M, int N, int K, hipStream_t s) {
  const long tiles_big = (long)ceil_div(M, 256) * ceil_div(N, 256);
  if (K % 32 == 0 && K >= 64) {  // both operands straight into LDS; tile choice as in gemm_f16 below
    if (direct_gemm_large_tiles(M, N)) {
      if (K % 64 == 0) return run_gemm_f16_bt_dma<Tile<256, 256, 128, 2, 4>, 2, OUT_F16>(a, bt, c, M, N, K, s);
      return run_gemm_f16_bt_dma<Tile<256, 256, 64, 2, 4>, 4, OUT_F16>(a, bt, c, M, N, K, s);
    }
    return run_gemm_f16_bt_dma<Tile<128, 128, 64, 2, 2>, 4, OUT_F16>(a, bt, c, M, N, K, s, direct_gemm_k_splits("UNIT_AMD_GEMM_F16_SPLITK", M, N, 2l * K));
  }
  if (M >= 256 && N >= 256 && tiles_big >= 128) return run_gemm_f16_bt<Tile<256, 256, 128, 2, 4>, OUT_F16>(a, bt, c, M, N, K, s);
  return run_gemm_f16_bt<Tile<128, 128, 64, 2, 2>, OUT_F16>(a, bt, c, M, N, K, s);
}

// b (K, N) -> bt (N, K): 64 x 64 tiles through LDS, 128-byte row segments on both sides
__global__ __launch_bounds__(256) void transpose_f16(const _Float16 *__restrict__ b, _Float16 *__restrict__ bt, int K,
                                                     int N) {
  __shared__ _Float16 tile[64][66];
  const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4)
    if (k0 + r < K && n0 + tx < N) tile[r][tx] = b[(size_t)(k0 + r) * N + n0 + tx];
  __syncthreads();
  for (int r = ty; r < 64; r += 4)
    if (n0 + r < N && k0 + tx < K) bt[(size_t)(n0 + r) * K + k0 + tx] = tile[tx][r];
}

// bp (N/32, K/32, 32, 32) with bp[y/32][k/32][k%32][y%32] = b[k][y] (apps/gpu/gemm-pack.py:9,17) -> bt (N, K):
// one 32 x 32 block (2 KiB, contiguous in bp) per workgroup, transposed through LDS; 64-byte row segments of bt
__global__ __launch_bounds__(256) void unpack32_f16(const _Float16 *__restrict__ bp, _Float16 *__restrict__ bt, int K) {
  __shared__ _Float16 tile[32][34];
  const int kb = blockIdx.x, nb = blockIdx.y;
  const _Float16 *src = bp + ((size_t)nb * gridDim.x + kb) * 1024;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int r = ty; r < 32; r += 8) tile[r][tx] = src[r * 32 + tx];  // tile[k % 32][y % 32]
  __syncthreads();
  for (int r = ty; r < 32; r += 8) bt[(size_t)(nb * 32 + r) * K + kb * 32 + tx] = tile[tx][r];
}

// TAIL = false: K is a whole number of stages (the loaders then stage without zeroing selects)
template <class T, bool OUT_F16, int PF = 1, bool TAIL = true>
int run_gemm_f16(const void *a, const void *b, void *c, int M, int N, int K, hipStream_t s) {
  using XL = RowMajorLoader<T::BX, T::BKB, T::NT, false, PF, TAIL>;
  using YL = KMajorF16Loader<T::BY, T::BKB, T::NT, PF, TAIL>;
  using Epi = GemmEpilogue<OpF16, OUT_F16>;
  typename XL::Params xp{static_cast<const char *>(a), M, K * 2, K * 2};
  typename YL::Params yp{static_cast<const char *>(b), N, K, N + 4, 0, N * 2};
  typename Epi::Params ep{c, M, N};
  const int nk = ceil_div(K * 2, T::BKB), gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
  const int splits = OUT_F16 ? 1 : gemm_k_splits("UNIT_AMD_GEMM_F16_SPLITK", M, N, 2l * K, nk);
  set_variant("f16gemm_x%d_y%d_k%d_w%dx%d_p%d%s%s_s%d", T::BX, T::BY, T::BKB, T::WX, T::WY, PF, TAIL ? "" : "e",
              OUT_F16 ? "_h" : "", splits);
  return launch_mma<OpF16, T, XL, YL, Epi, WS_NONE>(xp, yp, ep, nk, gx, gy, 4, splits, c, (size_t)M * N * 4, 0, s,
                                                    "unit_gemm_f16");
}

template <bool OUT_F16>
int gemm_f16(const void *a, const void *b, void *c, int M, int N, int K, hipStream_t s) {
  const long tiles_big = (long)ceil_div(M, 256) * ceil_div(N, 256);
  // UNIT_AMD_GEMM_F16_VARIANT pins a tile shape per process (measurement aid)
  switch (tuning_override("UNIT_AMD_GEMM_F16_VARIANT")) {
    case 1: return run_gemm_f16<Tile<256, 256, 128, 2, 4>, OUT_F16>(a, b, c, M, N, K, s);
    case 2: return run_gemm_f16<Tile<256, 256, 64, 2, 4>, OUT_F16>(a, b, c, M, N, K, s);
    case 3: return run_gemm_f16<Tile<256, 256, 128, 2, 2>, OUT_F16>(a, b, c, M, N, K, s);
    case 4: return K % 64 ? run_gemm_f16<Tile<256, 256, 128, 4, 2>, OUT_F16>(a, b, c, M, N, K, s)
                          : run_gemm_f16<Tile<256, 256, 128, 4, 2>, OUT_F16, 1, false>(a, b, c, M, N, K, s);
    case 5: return run_gemm_f16<Tile<256, 256, 64, 4, 2>, OUT_F16, 2>(a, b, c, M, N, K, s);
    case 6: return run_gemm_f16<Tile<128, 256, 128, 4, 2>, OUT_F16>(a, b, c, M, N, K, s);
    case 7: if (K % 64 == 0 && K >= 128) return run_gemm_f16_hybrid<Tile<256, 256, 128, 4, 2>, OUT_F16>(a, b, c, M, N, K, s); break;
    case 8: if (K % 64 == 0 && K >= 128) return run_gemm_f16_hybrid<Tile<256, 256, 128, 2, 4>, OUT_F16>(a, b, c, M, N, K, s); break;
    case 9: if (K % 64 == 0 && K >= 128) return run_gemm_f16_hybrid<Tile<256, 128, 128, 2, 2>, OUT_F16>(a, b, c, M, N, K, s); break;
    case 10: if (K % 64 == 0 && K >= 128 && N % 8 == 0) return run_gemm_f16_dma_tr<Tile<256, 256, 128, 2, 4>, 2, OUT_F16>(a, b, c, M, N, K, s); break;
    case 11: if (K % 32 == 0 && K >= 128 && N % 8 == 0) return run_gemm_f16_dma_tr<Tile<256, 256, 64, 2, 4>, 4, OUT_F16>(a, b, c, M, N, K, s); break;
    case 12: if (K % 32 == 0 && K >= 128 && N % 8 == 0) return run_gemm_f16_dma_tr<Tile<256, 128, 64, 2, 2>, 4, OUT_F16>(a, b, c, M, N, K, s); break;
    case 13: if (K % 32 == 0 && K >= 128 && N % 8 == 0) return run_gemm_f16_dma_tr<Tile<128, 256, 64, 2, 2>, 4, OUT_F16>(a, b, c, M, N, K, s); break;
    case 15: if (K % 32 == 0 && K >= 128 && N % 8 == 0) return run_gemm_f16_dma_tr<Tile<128, 128, 64, 2, 2>, 4, OUT_F16>(a, b, c, M, N, K, s); break;
    case 16: if (K % 32 == 0 && K >= 128 && N % 8 == 0) return run_gemm_f16_dma_tr<Tile<128, 128, 64, 2, 2>, 6, OUT_F16>(a, b, c, M, N, K, s); break;
    case 14: if (K % 32 == 0 && K >= 128 && N % 8 == 0) return run_gemm_f16_dma_tr<Tile<256, 128, 64, 2, 2>, 6, OUT_F16>(a, b, c, M, N, K, s); break;
    default: break;
  }
  // K a whole number of 64-byte stages and N of 16-byte chunks: both operands straight into LDS, b read back with the
  // transposing LDS read.  At 4096^3 116 us against 133 us for the register-transposing pipeline below, 2048^3 26
  // against 39 us, 1024 x 4096 x 4096 45 against 68 us, same bits.
  if (K % 32 == 0 && K >= 64 && N % 8 == 0) {
    if (direct_gemm_large_tiles(M, N)) {
      if (K % 64 == 0) return run_gemm_f16_dma_tr<Tile<256, 256, 128, 2, 4>, 2, OUT_F16>(a, b, c, M, N, K, s);
      return run_gemm_f16_dma_tr<Tile<256, 256, 64, 2, 4>, 4, OUT_F16>(a, b, c, M, N, K, s);
    }
    return run_gemm_f16_dma_tr<Tile<128, 128, 64, 2, 2>, 4, OUT_F16>(a, b, c, M, N, K, s, direct_gemm_k_splits("UNIT_AMD_GEMM_F16_SPLITK", M, N, 2l * K));
  }
  // K a whole number of 128-byte stages: a straight into LDS, b through the transposing register loader
  // (measured 130 us against 154 us for the all-register pipeline at 4096^3, same bits).  256 x 256 tiles of eight
  // waves, or 256 x 128 tiles of four when those need fewer rounds of 256 workgroups for their cost (about 0.55 of
  // a 256 x 256 tile: 2048^3 54 -> 36 us, 1024 x 4096 x 4096 95 -> 63 us, 8192 x 1024 x 1024 31 -> 25 us;
  // 3072^3 stays on 144 large tiles, 76 us, against 106 us on 288 small ones)
  if (M >= 256 && N >= 128 && K % 64 == 0 && K >= 128) {
    const long tiles_half = (long)ceil_div(M, 256) * ceil_div(N, 128);
    const long rounds_big = ceil_div((int)tiles_big, 256), rounds_half = ceil_div((int)tiles_half, 256);
    const bool big_ok = N >= 256 && tiles_big >= 128;
    if (big_ok && rounds_big * 100 <= rounds_half * 55)
      return run_gemm_f16_hybrid<Tile<256, 256, 128, 2, 4>, OUT_F16>(a, b, c, M, N, K, s);
    if (tiles_half >= 128) return run_gemm_f16_hybrid<Tile<256, 128, 128, 2, 2>, OUT_F16>(a, b, c, M, N, K, s);
    if (big_ok) return run_gemm_f16_hybrid<Tile<256, 256, 128, 2, 4>, OUT_F16>(a, b, c, M, N, K, s);
  }
  if (M >= 256 && N >= 256 && tiles_big >= 128) {
    // 64 (m) x 128 (n) wave tiles: measured 8-10 % faster than 128 x 64 (512-byte row runs per wave in the write-back)
    return run_gemm_f16<Tile<256, 256, 128, 4, 2>, OUT_F16>(a, b, c, M, N, K, s);
  }
  // mid sizes: 128 x 256 tiles of eight waves (measured 8-12 % faster than 128 x 128 at 2048^3, 1024 x 4096 x 4096)
  if (M >= 128 && N >= 256 && K >= 128) return run_gemm_f16<Tile<128, 256, 128, 4, 2>, OUT_F16>(a, b, c, M, N, K, s);
  return run_gemm_f16<Tile<128, 128, 64, 2, 2>, OUT_F16>(a, b, c, M, N, K, s);
}

// ---- k-splits through a workspace: plane s of the workspace takes the partial tiles of split s, a second kernel
// adds the planes in split order (deterministic; fp16 output rounds the final sum once)
using SplitTile = Tile<128, 128, 64, 2, 2>;

int gemm_f16_ws_splits(int M, int N, int K) {
  return gemm_k_splits("UNIT_AMD_GEMM_F16_SPLITK", M, N, 2l * K, ceil_div(K * 2, SplitTile::BKB));
}

template <bool OUT_F16>
__global__ __launch_bounds__(256) void add_planes(const v4f *__restrict__ ws, void *__restrict__ c, size_t n4, int splits,
                                                  size_t plane4) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  v4f sum = ws[i];
  for (int s = 1; s < splits; ++s) sum += ws[i + s * plane4];
  if constexpr (OUT_F16) {
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    static_cast<v4h *>(c)[i] = v4h{(_Float16)sum[0], (_Float16)sum[1], (_Float16)sum[2], (_Float16)sum[3]};
  } else {
    static_cast<v4f *>(c)[i] = sum;
  }
}

// a (M, K) . b (K, N) with `splits` > 1 k-ranges; ws holds splits * M * N floats
int gemm_f16_planes(const char *what, const void *a, const void *b, void *c, int M, int N, int K, bool out_f16, void *ws,
                    int splits, hipStream_t s) {
  using T = SplitTile;
  const size_t plane = (size_t)M * N * 4;
  GemmPlaneEpilogue::Params ep{ws, M, N, plane};
  if (K % 32 == 0 && N % 8 == 0 && splits <= K * 2 / T::BKB) {
    // whole 64-byte stages: both operands global -> LDS directly, b read back with the transposing LDS read
    if (int rc = run_gemm_f16_dma_tr<T, 4, GemmPlaneEpilogue>(what, out_f16 ? "planes_dmatr_h" : "planes_dmatr", a, b, ep, M, N,
                                                              K, splits, nullptr, s))
      return rc;
  } else {
    using XL = RowMajorLoader<T::BX, T::BKB, T::NT, false, 1, true>;
    using YL = KMajorF16Loader<T::BY, T::BKB, T::NT, 1, true>;
    typename XL::Params xp{static_cast<const char *>(a), M, K * 2, K * 2};
    typename YL::Params yp{static_cast<const char *>(b), N, K, N + 4, 0, N * 2};
    const int nk = ceil_div(K * 2, T::BKB), gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
    set_variant("f16gemm_planes_x%d_y%d_k%d_w%dx%d%s_s%d", T::BX, T::BY, T::BKB, T::WX, T::WY, out_f16 ? "_h" : "", splits);
    if (int rc = launch_mma<OpF16, T, XL, YL, GemmPlaneEpilogue, WS_NONE>(xp, yp, ep, nk, gx, gy, 4, splits, nullptr, 0, 0, s, what))
      return rc;
  }
  const size_t n4 = (size_t)M * N / 4;
  if (out_f16)
    hipLaunchKernelGGL(add_planes<true>, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, static_cast<const v4f *>(ws), c,
                       n4, splits, n4);
  else
    hipLaunchKernelGGL(add_planes<false>, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, static_cast<const v4f *>(ws),
                       c, n4, splits, n4);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
}

// argument checks shared by the entry points that split the reduction through planes; *splits = 1 when the shape
// runs without k-splits (then the plain entry point serves it)
int gemm_f16_ws_check(const char *what, const void *a, const void *b, const void *c, int M, int N, int K, int *splits) {
  if (!a || !b || !c) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (M <= 0 || N <= 0 || K <= 0) return fail(UNIT_E_ARG, "%s: M, N, K must be positive (got %d, %d, %d)", what, M, N, K);
  if (K % 8) return fail(UNIT_E_ARG, "%s: K must be a multiple of 8 (got %d)", what, K);
  if (N % 4) return fail(UNIT_E_ARG, "%s: N must be a multiple of 4 (got %d)", what, N);
  if (!fits((size_t)M * K * 2) || !fits((size_t)N * K * 2) || !fits((size_t)M * N * 4))
    return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  *splits = gemm_f16_ws_splits(M, N, K);
  return UNIT_OK;
}

}  // namespace
}  // namespace unit

// ---- the same planes in a buffer the library owns: a file-scope device array, so that the entry point below
// allocates nothing.  Each GPU the library runs on holds its own copy of the array at its own address, resolved once
// per device on the first call there (with that device current); host code uses that pointer, never the array's name.
namespace unit {
namespace {
constexpr size_t kStaticScratchBytes = 16u << 20;
static __device__ __align__(256) char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

int static_scratch(const char *what, void **ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(UNIT_E_DEVICE, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(UNIT_E_DEVICE, "%s: device index %d out of range", what, dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(UNIT_E_DEVICE, "%s: hipGetSymbolAddress: %s", what, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return UNIT_OK;
}
}  // namespace
}  // namespace unit

extern "C" int unit_gemm_f16_static(const void *a, const void *b, void *c, int32_t M, int32_t N, int32_t K, int32_t out_f16,
                                    unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_gemm_f16_static";
  int splits = 1;
  if (int rc = gemm_f16_ws_check(what, a, b, c, M, N, K, &splits)) return rc;
  if (int rc = check_aligned(what, {a, b, c})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (splits <= 1)  // nothing to split: no scratch is touched
    return out_f16 ? gemm_f16<true>(a, b, c, M, N, K, s) : gemm_f16<false>(a, b, c, M, N, K, s);
  const size_t need = (size_t)splits * M * N * 4;
  if (need > kStaticScratchBytes)
    return fail(UNIT_E_ARG, "%s: %d k-splits of %d x %d need %zu bytes of scratch, the static buffer holds %zu; "
                "use unit_gemm_f16_ws with a workspace", what, splits, M, N, need, kStaticScratchBytes);
  void *ws = nullptr;
  if (int rc = static_scratch(what, &ws)) return rc;
  // every plane element that add_planes reads is written by this call's GEMM first: nothing has to start at zero
  return gemm_f16_planes(what, a, b, c, M, N, K, out_f16 != 0, ws, splits, s);
}

extern "C" int unit_gemm_f16_ws_bytes(int32_t M, int32_t N, int32_t K, size_t *bytes) {
  using namespace unit;
  const char *what = "unit_gemm_f16_ws_bytes";
  if (!bytes) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (M <= 0 || N <= 0 || K <= 0 || K % 8 || N % 4)
    return fail(UNIT_E_ARG, "%s: M, N, K must be positive, K a multiple of 8 and N of 4 (got %d, %d, %d)", what, M, N, K);
  const int splits = gemm_f16_ws_splits(M, N, K);
  *bytes = splits > 1 ? (size_t)splits * M * N * 4 : 0;
  return UNIT_OK;
}

extern "C" int unit_gemm_f16_ws(const void *a, const void *b, void *c, int32_t M, int32_t N, int32_t K, int32_t out_f16,
                                void *workspace, size_t workspace_bytes, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_gemm_f16_ws";
  int splits = 1;
  if (int rc = gemm_f16_ws_check(what, a, b, c, M, N, K, &splits)) return rc;
  if (splits <= 1) {  // enough tiles, or a short reduction: nothing to split (the plain path makes the same choice)
    if (int rc = check_aligned(what, {a, b, c})) return rc;
    if (int rc = check_device()) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return out_f16 ? gemm_f16<true>(a, b, c, M, N, K, s) : gemm_f16<false>(a, b, c, M, N, K, s);
  }
  const size_t need = (size_t)splits * M * N * 4;
  if (!workspace || workspace_bytes < need)
    return fail(UNIT_E_ARG, "%s: workspace of %zu bytes needed (got %zu); ask unit_gemm_f16_ws_bytes", what, need,
                workspace ? workspace_bytes : (size_t)0);
  if (int rc = check_aligned(what, {a, b, c, workspace})) return rc;
  if (int rc = check_device()) return rc;
  return gemm_f16_planes(what, a, b, c, M, N, K, out_f16 != 0, workspace, splits, static_cast<hipStream_t>(stream));
}

extern "C" int unit_gemm_f16(const void *a, const void *b, void *c, int32_t M, int32_t N, int32_t K,
                             int32_t out_f16, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_gemm_f16";
  if (!a || !b || !c) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (M <= 0 || N <= 0 || K <= 0) return fail(UNIT_E_ARG, "%s: M, N, K must be positive (got %d, %d, %d)", what, M, N, K);
  if (K % 8) return fail(UNIT_E_ARG, "%s: K must be a multiple of 8 (got %d)", what, K);
  if (N % 4) return fail(UNIT_E_ARG, "%s: N must be a multiple of 4 (got %d)", what, N);
  if (const int per = row_slice(M, (size_t)K * 2, (size_t)N * 4))
    return run_row_slices(M, per, (size_t)K * 2, (size_t)N * (out_f16 ? 2 : 4), a, c, [&](const void *as, void *cs, int rows) {
      return unit_gemm_f16(as, b, cs, rows, N, K, out_f16, stream);
    });
  if (!fits((size_t)M * K * 2) || !fits((size_t)N * K * 2) || !fits((size_t)M * N * 4))
    return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {a, b, c})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return out_f16 ? gemm_f16<true>(a, b, c, M, N, K, s) : gemm_f16<false>(a, b, c, M, N, K, s);
}

extern "C" int unit_gemm_f16_prepare_b(const void *b, void *bt, int32_t K, int32_t N, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_gemm_f16_prepare_b";
  if (!b || !bt) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (K <= 0 || N <= 0) return fail(UNIT_E_ARG, "%s: K, N must be positive (got %d, %d)", what, K, N);
  if (K % 8) return fail(UNIT_E_ARG, "%s: K must be a multiple of 8 (got %d)", what, K);
  if (!fits((size_t)N * K * 2)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {b, bt})) return rc;
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(transpose_f16, dim3(ceil_div(N, 64), ceil_div(K, 64)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const _Float16 *>(b), static_cast<_Float16 *>(bt), K, N);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  set_variant("f16_transpose_b");
  return UNIT_OK;
}

extern "C" int unit_gemm_f16_prepare_b_packed32(const void *bp, void *bt, int32_t K, int32_t N, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_gemm_f16_prepare_b_packed32";
  if (!bp || !bt) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (K <= 0 || N <= 0) return fail(UNIT_E_ARG, "%s: K, N must be positive (got %d, %d)", what, K, N);
  if (K % 32 || N % 32) return fail(UNIT_E_ARG, "%s: K and N must be multiples of 32 (got %d, %d)", what, K, N);
  if (!fits((size_t)N * K * 2)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (N / 32 > 65535) return fail(UNIT_E_ARG, "%s: N exceeds 32 * 65535", what);
  if (int rc = check_aligned(what, {bp, bt})) return rc;
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(unpack32_f16, dim3(K / 32, N / 32), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const _Float16 *>(bp), static_cast<_Float16 *>(bt), K);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  set_variant("f16_unpack32_b");
  return UNIT_OK;
}

extern "C" int unit_gemm_f16_prepared(const void *a, const void *bt, void *c, int32_t M, int32_t N, int32_t K,
                                      int32_t out_f16, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_gemm_f16_prepared";
  if (!a || !bt || !c) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (M <= 0 || N <= 0 || K <= 0) return fail(UNIT_E_ARG, "%s: M, N, K must be positive (got %d, %d, %d)", what, M, N, K);
  if (K % 8) return fail(UNIT_E_ARG, "%s: K must be a multiple of 8 (got %d)", what, K);
  if (N % 4) return fail(UNIT_E_ARG, "%s: N must be a multiple of 4 (got %d)", what, N);
  if (const int per = row_slice(M, (size_t)K * 2, (size_t)N * 4))
    return run_row_slices(M, per, (size_t)K * 2, (size_t)N * (out_f16 ? 2 : 4), a, c, [&](const void *as, void *cs, int rows) {
      return unit_gemm_f16_prepared(as, bt, cs, rows, N, K, out_f16, stream);
    });
  if (!fits((size_t)M * K * 2) || !fits((size_t)N * K * 2) || !fits((size_t)M * N * 4))
    return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {a, bt, c})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return out_f16 ? gemm_f16_bt<true>(a, bt, c, M, N, K, s) : gemm_f16_bt<false>(a, bt, c, M, N, K, s);
}
