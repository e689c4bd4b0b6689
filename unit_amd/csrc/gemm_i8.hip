// int8 dense: c (M, N) i32 = a (M, K) u8 . W^T, W s8 given row-major (N, K) or in the reference's
// (N/128, K/4, 128, 4) pre-pack.  X operand = a (rows m), Y operand = W (rows n).
#include "epilogues.hpp"
#include "host.hpp"
#include "loaders.hpp"
#include "gemm_mixed.hpp"
#include "mma_dma.hpp"

namespace unit {
namespace {

// TAIL = false: K is a whole number of stages (the loaders then stage without zeroing selects)
template <class T, bool PACKED, bool TAIL = true>
int run_dense(const void *a, const void *w, void *c, int M, int N, int K, hipStream_t s) {
  using XL = RowMajorLoader<T::BX, T::BKB, T::NT, true, 1, TAIL>;
  using YLrm = RowMajorLoader<T::BY, T::BKB, T::NT, false, 1, TAIL>;
  using YLpk = VnniLoader<T::BY, T::BKB, T::NT, 128, 1, TAIL>;
  using Epi = GemmEpilogue<OpI8, false>;
  typename XL::Params xp{static_cast<const char *>(a), M, K, K};
  typename Epi::Params ep{c, M, N};
  const int nk = ceil_div(K, T::BKB), gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
  // few tiles and a long reduction: share K between workgroups (int32 atomics are exact)
  int splits = gemm_k_splits("UNIT_AMD_DENSE_SPLITK", M, N, K, nk);
  if ((size_t)M * N * 4 % 16) splits = 1;
  set_variant("i8dense%s_x%d_y%d_k%d_w%d%s_s%d", PACKED ? "pk" : "rm", T::BX, T::BY, T::BKB, T::NT / 64, TAIL ? "" : "e",
              splits);
  if constexpr (PACKED) {
    typename YLpk::Params yp{static_cast<const char *>(w), N, K / 4};
    return launch_mma<OpI8, T, XL, YLpk, Epi, WS_Y>(xp, yp, ep, nk, gx, gy, 4, splits, c, (size_t)M * N * 4, 0, s,
                                                    "unit_dense_dotprod_u8s8s32");
  } else {
    typename YLrm::Params yp{static_cast<const char *>(w), N, K, K};
    return launch_mma<OpI8, T, XL, YLrm, Epi, WS_Y>(xp, yp, ep, nk, gx, gy, 4, splits, c, (size_t)M * N * 4, 0, s,
                                                    "unit_dense_u8s8s32");
  }
}

// direct-to-LDS variant: row-major weights, K a whole number of stages.  wsum: the weight's row sums when they
// were prepared beforehand (unit_dense_prepare_weight), else null and the kernel sums the fragments itself -- one
// Y block per wave where the tile has as many Y blocks per wave as waves share them (WS_Y_SPLIT: 4096^3 in 66-69 us
// against 65 us on prepared sums; summing every fragment in every wave cost 75 us).
template <class T, int NSTAGE, bool GIVEN = false>
int run_dense_dma(const void *a, const void *w, void *c, int M, int N, int K, hipStream_t s, const int *wsum = nullptr,
                  int splits = 1) {
  using Epi = GemmEpilogue<OpI8, false>;
  DmaParams p{static_cast<const char *>(a), static_cast<const char *>(w), M, N, K, wsum};
  typename Epi::Params ep{c, M, N};
  const int nk = K / T::BKB, gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
  constexpr int lds = NSTAGE * T::STAGE;
  static_assert(lds <= kMaxLds, "ring does not fit the LDS");
  constexpr bool kSplitSums = !GIVEN && T::TY == T::WX && (T::TY & (T::TY - 1)) == 0 && T::TX * T::TY >= 6;
  auto kern = mma_dma_kernel<OpI8, T, NSTAGE, Epi, GIVEN ? WS_Y_GIVEN : kSplitSums ? WS_Y_SPLIT : WS_Y, true>;
  static thread_local bool allowed = false;
  if (!allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "unit_dense_u8s8s32: hipFuncSetAttribute: %s", hipGetErrorString(e));
    allowed = true;
  }
  splits = splits < 1 || (size_t)M * N * 4 % 16 ? 1 : (splits > nk ? nk : splits);
  if (splits > 1) {  // the k-ranges add into c with atomics (exact for int32)
    const size_t n16 = (size_t)M * N * 4 / 16;
    hipLaunchKernelGGL(zero_fill, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, s, static_cast<v4i *>(c), n16);
  }
  const GridMap gm = GridMap::make(gx, gy, gx < 4 ? gx : 4, splits);
  set_variant("i8dense%sdma_x%d_y%d_k%d_w%dx%d_r%d_s%d", GIVEN ? "prep_" : "", T::BX, T::BY, T::BKB, T::WX, T::WY, NSTAGE,
              splits);
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(T::NT), lds, s, p, ep, nk, gm UNIT_TRACE(, trace_buffer()));
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "unit_dense_u8s8s32: launch: %s", hipGetErrorString(e));
}

// pre-packed weights straight to registers, activations through LDS (UNIT_AMD_DENSE_VARIANT=13).
// Measured equal to the staged kernel (91.6 vs 91.1 us at 4096^3) although it moves 1.6 x less
// through LDS: the GEMM is bound by instruction issue per SIMD, not by the LDS pipe.
int run_dense_mixed(const void *a, const void *wp, void *c, int M, int N, int K, hipStream_t s) {
  using T = Tile<256, 256, 128, 2, 4>;
  using XL = RowMajorLoader<T::BX, T::BKB, T::NT, true>;
  using Epi = GemmEpilogue<OpI8, false>;
  const char *what = "unit_dense_dotprod_u8s8s32";
  typename XL::Params xp{static_cast<const char *>(a), M, K, K};
  typename Epi::Params ep{c, M, N};
  const int nk = ceil_div(K, T::BKB), gx = ceil_div(M, T::BX), gy = ceil_div(N, T::BY);
  constexpr int lds = 2 * T::XBYTES;
  auto kern = gemm_mixed_i8<T>;
  static thread_local bool allowed = false;
  if (!allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
    if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
    allowed = true;
  }
  const GridMap gm = GridMap::make(gx, gy, gx < 4 ? gx : 4, 1);
  set_variant("i8densepk_direct_x%d_y%d_k%d_w%d_s1", T::BX, T::BY, T::BKB, T::NT / 64);
  hipLaunchKernelGGL(kern, dim3(gm.total), dim3(T::NT), lds, s, xp, static_cast<const char *>(wp), N, K / 4, ep, nk, gm);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? UNIT_OK : fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
}

template <bool PACKED>
int dense(const void *a, const void *w, void *c, int M, int N, int K, unit_stream_t stream) {
  const char *what = PACKED ? "unit_dense_dotprod_u8s8s32" : "unit_dense_u8s8s32";
  if (!a || !w || !c) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (M <= 0 || N <= 0 || K <= 0) return fail(UNIT_E_ARG, "%s: M, N, K must be positive (got %d, %d, %d)", what, M, N, K);
  if (K % 16) return fail(UNIT_E_ARG, "%s: K must be a multiple of 16 (got %d)", what, K);
  if (PACKED && N % 128) return fail(UNIT_E_ARG, "%s: N must be a multiple of 128 (got %d)", what, N);
  if (!PACKED && N % 4) return fail(UNIT_E_ARG, "%s: N must be a multiple of 4 (got %d)", what, N);
  if (const int per = row_slice(M, (size_t)K, (size_t)N * 4))
    return run_row_slices(M, per, (size_t)K, (size_t)N * 4, a, c, [&](const void *as, void *cs, int rows) {
      return dense<PACKED>(as, w, cs, rows, N, K, stream);
    });
  if (!fits((size_t)M * K) || !fits((size_t)N * K) || !fits((size_t)M * N * 4))
    return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {a, w, c})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long tiles_big = (long)ceil_div(M, 256) * ceil_div(N, 256);
  switch (tuning_override("UNIT_AMD_DENSE_VARIANT")) {
    case 1: return run_dense<Tile<256, 256, 128, 2, 2>, PACKED>(a, w, c, M, N, K, s);
    case 2: return run_dense<Tile<256, 256, 64, 2, 4>, PACKED>(a, w, c, M, N, K, s);
    case 3: return run_dense<Tile<256, 128, 64, 2, 2>, PACKED>(a, w, c, M, N, K, s);
    case 4: return run_dense<Tile<128, 128, 64, 2, 2>, PACKED>(a, w, c, M, N, K, s);
    case 5: return run_dense<Tile<256, 256, 64, 2, 2>, PACKED>(a, w, c, M, N, K, s);
    case 6: return run_dense<Tile<128, 256, 128, 1, 4>, PACKED>(a, w, c, M, N, K, s);
    case 7: if (!PACKED && K % 64 == 0) return run_dense_dma<Tile<256, 256, 64, 2, 2>, 4>(a, w, c, M, N, K, s); break;
    case 8: if (!PACKED && K % 64 == 0) return run_dense_dma<Tile<256, 256, 64, 2, 4>, 4>(a, w, c, M, N, K, s); break;
    case 9: if (!PACKED && K % 128 == 0) return run_dense_dma<Tile<256, 256, 128, 2, 2>, 2>(a, w, c, M, N, K, s); break;
    case 10: if (!PACKED && K % 64 == 0) return run_dense_dma<Tile<256, 256, 64, 2, 2>, 3>(a, w, c, M, N, K, s); break;
    case 11: if (!PACKED && K % 64 == 0) return run_dense_dma<Tile<256, 128, 64, 2, 2>, 4>(a, w, c, M, N, K, s); break;
    case 12: if (!PACKED && K % 128 == 0) return run_dense_dma<Tile<256, 256, 128, 2, 4>, 2>(a, w, c, M, N, K, s); break;
    case 13: if (PACKED) return run_dense_mixed(a, w, c, M, N, K, s); break;
    case 14: return run_dense<Tile<256, 256, 128, 2, 4>, PACKED>(a, w, c, M, N, K, s);
    case 15: return run_dense<Tile<256, 256, 128, 4, 2>, PACKED>(a, w, c, M, N, K, s);
    case 16: if (!PACKED && K % 128 == 0) return run_dense_dma<Tile<256, 256, 128, 4, 2>, 2>(a, w, c, M, N, K, s); break;
    case 17: if (!PACKED && K % 64 == 0) return run_dense_dma<Tile<128, 128, 64, 2, 2>, 4>(a, w, c, M, N, K, s); break;
    default: break;
  }
  // row-major weights, K a whole number of 64-byte stages, and a shape that 128 x 128 tiles fill better than 256 x 256
  // ones: both operands global -> LDS directly, two workgroups per CU (2048^3 23.3 -> 20.7 us, 1024 x 4096 x 4096
  // 39.8 -> 32.7 us, 8192 x 1024 x 1024 24.6 -> 18.0 us)
  if (!PACKED && K % 64 == 0 && !direct_gemm_large_tiles(M, N))
    return run_dense_dma<Tile<128, 128, 64, 2, 2>, 4>(a, w, c, M, N, K, s, nullptr,
                                                      direct_gemm_k_splits("UNIT_AMD_DENSE_SPLITK", M, N, K));
  // the large tiles on the same pipeline: the four waves that share a weight fragment divide the weight sums
  if (!PACKED && K % 128 == 0 && direct_gemm_large_tiles(M, N))
    return run_dense_dma<Tile<256, 256, 128, 4, 2>, 2>(a, w, c, M, N, K, s);
  if (M >= 256 && N >= 256 && tiles_big >= 128)
    return K % 128 ? run_dense<Tile<256, 256, 128, 2, 4>, PACKED>(a, w, c, M, N, K, s)
                   : run_dense<Tile<256, 256, 128, 2, 4>, PACKED, false>(a, w, c, M, N, K, s);
  return run_dense<Tile<128, 128, 64, 2, 2>, PACKED>(a, w, c, M, N, K, s);
}

// one wave per weight row: sum of its K bytes
__global__ __launch_bounds__(256) void dense_row_sums(const char *__restrict__ w, int *__restrict__ sums, int N, int K) {
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= N) return;
  const int *row = reinterpret_cast<const int *>(w + (size_t)n * K);
  int s = 0;
  for (int i = lane; i < K / 4; i += 64) s = __builtin_amdgcn_sdot4(row[i], 0x01010101, s, false);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) sums[n] = s;
}

}  // namespace
}  // namespace unit

extern "C" int unit_dense_prepare_weight(const void *w, int32_t *wsum, int32_t N, int32_t K, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_dense_prepare_weight";
  if (!w || !wsum) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (N <= 0 || K <= 0 || K % 16) return fail(UNIT_E_ARG, "%s: N, K must be positive and K a multiple of 16 (got %d, %d)", what, N, K);
  if (!fits((size_t)N * K)) return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {w})) return rc;
  if (int rc = check_device()) return rc;
  hipLaunchKernelGGL(dense_row_sums, dim3(ceil_div(N, 4)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const char *>(w), wsum, N, K);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(UNIT_E_LAUNCH, "%s: launch: %s", what, hipGetErrorString(e));
  set_variant("dense_row_sums_n%d_k%d", N, K);
  return UNIT_OK;
}

extern "C" int unit_dense_u8s8s32_prepared(const void *a, const void *w, const int32_t *wsum, void *c, int32_t M, int32_t N,
                                           int32_t K, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_dense_u8s8s32_prepared";
  if (!a || !w || !wsum || !c) return fail(UNIT_E_ARG, "%s: null pointer", what);
  // the direct-to-LDS kernels need whole stages (128 bytes for the 256 x 256 tiles, 64 for the 128 x 128 ones);
  // everything else runs the plain entry point, which sums the weights itself (same result)
  const bool large = M > 0 && N > 0 && direct_gemm_large_tiles(M, N);
  if (M <= 0 || N <= 0 || K <= 0 || K % (large ? 128 : 64) || N % 4 || row_slice(M, (size_t)K, (size_t)N * 4) ||
      !fits((size_t)M * K) || !fits((size_t)N * K) || !fits((size_t)M * N * 4))
    return unit_dense_u8s8s32(a, w, c, M, N, K, stream);
  if (int rc = check_aligned(what, {a, w, c})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (large) return run_dense_dma<Tile<256, 256, 128, 4, 2>, 2, true>(a, w, c, M, N, K, s, wsum);
  return run_dense_dma<Tile<128, 128, 64, 2, 2>, 4, true>(a, w, c, M, N, K, s, wsum,
                                                          direct_gemm_k_splits("UNIT_AMD_DENSE_SPLITK", M, N, K));
}

extern "C" int unit_dense_dotprod_u8s8s32(const void *a, const void *wp, void *c, int32_t M, int32_t N, int32_t K,
                                          unit_stream_t stream) {
  return unit::dense<true>(a, wp, c, M, N, K, stream);
}

extern "C" int unit_dense_u8s8s32(const void *a, const void *w, void *c, int32_t M, int32_t N, int32_t K,
                                  unit_stream_t stream) {
  return unit::dense<false>(a, w, c, M, N, K, stream);
}
