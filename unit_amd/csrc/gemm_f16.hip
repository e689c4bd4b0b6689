// fp16 GEMM: c (M, N) = a (M, K) f16 . b (K, N) f16, fp32 accumulate on v_mfma_f32_32x32x16_f16.
// X operand = a (rows m, K-contiguous), Y operand = b (rows n, transposed while staging).
#include "epilogues.hpp"
#include "host.hpp"
#include "loaders.hpp"

namespace unit {
namespace {

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
  set_variant("f16gemm_x%d_y%d_k%d_w%dx%d_p%d%s%s", T::BX, T::BY, T::BKB, T::WX, T::WY, PF, TAIL ? "" : "e",
              OUT_F16 ? "_h" : "");
  return launch_mma<OpF16, T, XL, YL, Epi, WS_NONE>(xp, yp, ep, nk, gx, gy, 4, 1, c, 0, 0, s, "unit_gemm_f16");
}

template <bool OUT_F16>
int gemm_f16(const void *a, const void *b, void *c, int M, int N, int K, hipStream_t s) {
  const long tiles_big = (long)ceil_div(M, 256) * ceil_div(N, 256);
  // UNIT_AMD_GEMM_F16_VARIANT pins a tile shape per process (measurement aid)
  switch (tuning_override("UNIT_AMD_GEMM_F16_VARIANT")) {
    case 1: return run_gemm_f16<Tile<256, 256, 128, 2, 4>, OUT_F16>(a, b, c, M, N, K, s);
    case 2: return run_gemm_f16<Tile<256, 256, 64, 2, 4>, OUT_F16>(a, b, c, M, N, K, s);
    case 3: return run_gemm_f16<Tile<256, 256, 128, 2, 2>, OUT_F16>(a, b, c, M, N, K, s);
    case 4: return run_gemm_f16<Tile<256, 256, 128, 4, 2>, OUT_F16>(a, b, c, M, N, K, s);
    case 5: return run_gemm_f16<Tile<256, 256, 64, 4, 2>, OUT_F16, 2>(a, b, c, M, N, K, s);
    case 6: return run_gemm_f16<Tile<128, 256, 128, 4, 2>, OUT_F16>(a, b, c, M, N, K, s);
    default: break;
  }
  // 64 (m) x 128 (n) wave tiles: measured 8-10 % faster than 128 x 64 (512-byte row runs per wave in the write-back)
  if (M >= 256 && N >= 256 && tiles_big >= 128)
    return K % 64 ? run_gemm_f16<Tile<256, 256, 128, 4, 2>, OUT_F16>(a, b, c, M, N, K, s)
                  : run_gemm_f16<Tile<256, 256, 128, 4, 2>, OUT_F16, 1, false>(a, b, c, M, N, K, s);
  return run_gemm_f16<Tile<128, 128, 64, 2, 2>, OUT_F16>(a, b, c, M, N, K, s);
}

}  // namespace
}  // namespace unit

extern "C" int unit_gemm_f16(const void *a, const void *b, void *c, int32_t M, int32_t N, int32_t K,
                             int32_t out_f16, unit_stream_t stream) {
  using namespace unit;
  const char *what = "unit_gemm_f16";
  if (!a || !b || !c) return fail(UNIT_E_ARG, "%s: null pointer", what);
  if (M <= 0 || N <= 0 || K <= 0) return fail(UNIT_E_ARG, "%s: M, N, K must be positive (got %d, %d, %d)", what, M, N, K);
  if (K % 8) return fail(UNIT_E_ARG, "%s: K must be a multiple of 8 (got %d)", what, K);
  if (N % 4) return fail(UNIT_E_ARG, "%s: N must be a multiple of 4 (got %d)", what, N);
  if (!fits((size_t)M * K * 2) || !fits((size_t)N * K * 2) || !fits((size_t)M * N * 4))
    return fail(UNIT_E_ARG, "%s: tensor exceeds 2^31-1 bytes", what);
  if (int rc = check_aligned(what, {a, b, c})) return rc;
  if (int rc = check_device()) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return out_f16 ? gemm_f16<true>(a, b, c, M, N, K, s) : gemm_f16<false>(a, b, c, M, N, K, s);
}
