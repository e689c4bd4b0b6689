/*
 * unit_amd -- C ABI of the MI355X (gfx950) tensorized conv2d / dense / GEMM path.
 *
 * The reference has no FFI of its own: its operators are Python functions on TVM
 * tensors.  Each entry point below names the reference operator (file:line, relative to
 * the reference tree) whose arithmetic it replaces; a binding only has to pass device
 * pointers and the operator's own shape arguments.
 *
 * Conventions
 *   - every pointer is a device pointer owned by the caller; the library never
 *     allocates or frees device memory and keeps no state between calls;
 *   - `stream` is a hipStream_t (NULL = default stream); calls enqueue work and return
 *     without synchronising;
 *   - return value 0 = enqueued; <0 = rejected (UNIT_E_*), nothing enqueued, and
 *     unit_last_error() returns a thread-local message;
 *   - int8 results are exact (int32 accumulation, wrapping mod 2^32 like vpdpbusd);
 *     fp16 inputs are multiplied and accumulated in fp32 on the MFMA unit;
 *   - a tensor may not exceed 2^31-1 bytes; the activations of the convolutions and of the
 *     layout kernels may, as long as a single image stays below: such a call runs as several
 *     launches over slices of the batch; likewise a and c of the GEMMs, over slices of rows.
 */
#ifndef UNIT_AMD_H
#define UNIT_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define UNIT_OK 0
#define UNIT_E_ARG (-1)     /* bad shape / null pointer / unsupported combination */
#define UNIT_E_LAUNCH (-2)  /* HIP refused the launch */
#define UNIT_E_DEVICE (-3)  /* current device is not gfx950 */

typedef void *unit_stream_t;

/* ABI version (major * 100 + minor). */
int unit_version(void);
/* Message for the last non-zero return on this thread ("" if none). */
const char *unit_last_error(void);
/* Name of the kernel variant the last successful compute call on this thread enqueued
 * (e.g. "i8conv_x256_y256_k128_w8"): the analogue of the tuned-schedule index the reference
 * logs per shape (python/tensorizer/tune.py:20-31). */
const char *unit_last_variant(void);
/* Number of tile variants the convolution entry points hold; the environment variable
 * UNIT_AMD_CONV_VARIANT=1..count pins one per process, as the reference pins a schedule index
 * through the tensorizer.tune globals (python/tensorizer/tune.py:3-16). */
int unit_conv_variant_count(void);
/* 1 if variant 0..count-1 takes its operands straight from global memory into MFMA fragments
 * (prepared weights or the reference's layout), 2 if it shares both operand tiles through LDS by
 * direct global -> LDS loads (convolutions on prepared weights, 16-channel blocks only), 0 if
 * it stages them in LDS through registers (the reference's weight layout only), -1 if there is no
 * such variant.  For the tuner; no counterpart in the reference. */
int unit_conv_variant_is_direct(int32_t variant);

/* Geometry of one 2-D convolution; C and K are the channel counts as stored in the blocked
 * tensors (already rounded up: C % cb == 0, K % 16 == 0, apps/cpu/kernel/conv2d.py:18-22). */
typedef struct unit_conv_desc {
  int32_t N, C, H, W; /* data: batch, input channels, height, width (unpadded) */
  int32_t K, KH, KW;  /* output channels, kernel height, width */
  int32_t sh, sw;     /* strides */
  int32_t pt, pl, pb, pr; /* zero padding: top, left, bottom, right */
  int32_t dh, dw;     /* dilation */
  int32_t cb;         /* input-channel block of the data layout: 16 or 4 (int8); 16 (fp16) */
} unit_conv_desc;

/* Output height/width for a descriptor; UNIT_E_ARG if the window does not fit. */
int unit_conv_out_hw(const unit_conv_desc *d, int32_t *OH, int32_t *OW);

/* ------------------------------------------------------------------ int8 compute */

/* topi.nn.conv2d_NCHWc_int8(data, kernel, stride, padding, dilation, out_dtype='int32',
 * layout='NCHW{cb}c', out_layout='NCHW16c') as called at apps/cpu/kernel/conv2d.py:50-51
 * (closed form: apps/cpu/kernel/conv3d.py:60-64).
 *   data   u8  (N, C/cb, H, W, cb)
 *   weight s8  (K/16, C/cb, KH, KW, cb/4, 16, 4)       -- the reference's VNNI pre-pack
 *   out    i32 (N, K/16, OH, OW, 16)
 * u8 x s8 -> i32, replacing llvm.x86.avx512.vpdpbusd.512
 * (python/tensorizer/intrinsics/cpu.py:42-49,189-193) with v_mfma_i32_32x32x32_i8. */
int unit_conv2d_nchwc_u8s8s32(const unit_conv_desc *d, const void *data, const void *weight,
                              void *out, unit_stream_t stream);

/* The convolution as the reference's quantized models run it,
 * fused_nn_contrib_conv2d_NCHWc_subtract_add_multiply (apps/cpu/relay/result.log:3-26,35):
 * signed activations x are shifted to u8 (x + 128), convolved, corrected by 128 * sum(w) per
 * output channel, biased and scaled:
 *   out = (conv_u8(x + 128, w) - 128 * sum_{c,kh,kw} w[k] + bias[k]) * scale      (all int32)
 * which equals (sum x * w + bias[k]) * scale on the signed data; the signed MFMA computes that
 * directly, with neither the shift nor the correction.
 *   data   s8  (N, C/cb, H, W, cb)
 *   weight s8  (K/16, C/cb, KH, KW, cb/4, 16, 4)
 *   bias   i32 (K) or NULL;  scale: int32 factor (the reference prints 11)
 *   out    i32 (N, K/16, OH, OW, 16) */
int unit_conv2d_nchwc_s8s8s32_fused(const unit_conv_desc *d, const void *data, const void *weight,
                                    const int32_t *bias, int32_t scale, void *out, unit_stream_t stream);

/* 3-D convolution of apps/cpu/kernel/conv3d.py:39-64 (the reference's only closed form of the
 * blocked convolution): valid (no padding), one stride for the three dimensions, s8 x s8 -> i32
 * as its te.compute casts both operands from int8:
 *   O[n,ko,x,y,z,kb] = sum_{ci,rd,rh,rw,e,i} A[n,ci,s*x+rd,s*y+rh,s*z+rw,4e+i] * W[ko,ci,rd,rh,rw,e,kb,i]
 *   data   s8  (N, C/cb, D, H, W, cb)
 *   weight s8  (K/16, C/cb, KD, KH, KW, cb/4, 16, 4)
 *   out    i32 (N, K/16, OD, OH, OW, 16),  O* = (* - K*) / stride + 1
 * The channel block follows conv3d.py:39-56: cb = 16 when C is a multiple of 16, else 4 (C a
 * multiple of 4; KW <= 8 and KH <= 31 then: its 3 -> 4 channel 7x7x7 workload, conv3d.py:22). */
typedef struct unit_conv3d_desc {
  int32_t N, C, D, H, W; /* data: batch, input channels (multiple of 4), depth, height, width */
  int32_t K, KD, KH, KW; /* output channels (multiple of 16), kernel depth, height, width */
  int32_t stride;
} unit_conv3d_desc;
int unit_conv3d_ncdhwc_s8s8s32(const unit_conv3d_desc *d, const void *data, const void *weight, void *out,
                               unit_stream_t stream);

/* topi.x86.dense_dotprod(data, weight, None, 'int32') as called at
 * apps/cpu/kernel/int8-gemm.py:13-16.
 *   a   u8  (M, K) row-major
 *   wp  s8  (N/128, K/4, 128, 4),  wp[n/128][k/4][n%128][k%4] = W[n][k]
 *   c   i32 (M, N) = a . W^T
 * N % 128 == 0, K % 16 == 0. */
int unit_dense_dotprod_u8s8s32(const void *a, const void *wp, void *c, int32_t M, int32_t N,
                               int32_t K, unit_stream_t stream);

/* relay.nn.dense(x, w, out_dtype='int32') of apps/cpu/relay/int8-gemm.py:14-16 on the
 * un-packed weight:  a u8 (M, K), w s8 (N, K) row-major, c i32 (M, N) = a . w^T.
 * K % 16 == 0.  Few output tiles: the reduction is split between workgroups (int32 atomics, exact). */
int unit_dense_u8s8s32(const void *a, const void *w, void *c, int32_t M, int32_t N, int32_t K,
                       unit_stream_t stream);

/* The same dense with the constant part of the u8 -> s8 shift folded once per weight, as the reference's
 * compiled graphs fold sum(w) next to their u8 x s8 operators (apps/cpu/relay/result.log:15-16 for the
 * convolution; the dense weight of apps/cpu/relay/int8-gemm.py:15 is a constant the same way):
 *   unit_dense_prepare_weight  wsum[n] = sum_k w[n][k]  (int32[N], caller-owned)
 *   unit_dense_u8s8s32_prepared  c = a . w^T with both operand tiles moved global -> LDS directly (K % 128 == 0
 *   and at least 128 tiles of 256 x 256; other shapes run unit_dense_u8s8s32).  Results are identical. */
int unit_dense_prepare_weight(const void *w, int32_t *wsum, int32_t N, int32_t K, unit_stream_t stream);
int unit_dense_u8s8s32_prepared(const void *a, const void *w, const int32_t *wsum, void *c, int32_t M,
                                int32_t N, int32_t K, unit_stream_t stream);

/* ------------------------------------------------------------------ fp16 compute */

/* The fp16 GEMM of apps/gpu/gemm.py:8-20 (CUDA form: poc/tensorcore/gemm-prefetch.cu:66-164):
 *   c[x][y] = sum_k f32(a[x][k]) * f32(b[k][y]),  a f16 (M, K), b f16 (K, N), row-major;
 * c is f32 when out_f16 == 0, else f16 (round-to-nearest-even of the fp32 sum).
 * K % 8 == 0, N % 4 == 0.  Replaces wmma.m16n16k16 (python/tensorizer/intrinsics/gpu.py:104-216)
 * with v_mfma_f32_32x32x16_f16.  With few output tiles and a long reduction (the script's own
 * 128 x 768 x 3072) and f32 output, the reduction is split between workgroups as the reference's
 * rfactor schedule does (apps/gpu/gemm.py:22-40): partial tiles are added into the zero-filled c,
 * so the summation order, and with it the last bits of c, can differ from run to run
 * (UNIT_AMD_GEMM_F16_SPLITK=1 keeps one workgroup per tile). */
int unit_gemm_f16(const void *a, const void *b, void *c, int32_t M, int32_t N, int32_t K,
                  int32_t out_f16, unit_stream_t stream);

/* The same GEMM with the k-splits' partial tiles kept apart: split s writes plane s (M * N floats) of a
 * caller-owned workspace and a second kernel adds the planes in split order, as the reference's host
 * check adds its split-K partial sums in a fixed order (poc/tensorcore/gemm-prefetch.cu:213-228).  The result no
 * longer depends on which workgroup finishes first (bit-identical from run to run), and f16 output can use the
 * k-splits too (the sum is rounded once).  unit_gemm_f16_ws_bytes gives the workspace size for a shape: 0 when
 * the shape has enough output tiles, or too short a reduction, to run without k-splits (then workspace may be
 * null and the call is unit_gemm_f16 with one workgroup per tile).  Same argument rules as unit_gemm_f16;
 * M * N * 4 bytes <= 2^31 - 1. */
int unit_gemm_f16_ws_bytes(int32_t M, int32_t N, int32_t K, size_t *bytes);
int unit_gemm_f16_ws(const void *a, const void *b, void *c, int32_t M, int32_t N, int32_t K, int32_t out_f16,
                     void *workspace, size_t workspace_bytes, unit_stream_t stream);

/* unit_gemm_f16_ws without the workspace argument: the planes live in a 16 MiB device array inside the library, so
 * the call allocates nothing (no hipMalloc / hipFree, here or in anything it calls).  It has no counterpart in the
 * reference; it is for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses
 * that forbid allocation.  Same results as unit_gemm_f16_ws, bit for bit.  Shapes whose k-splits need more than
 * 16 MiB (splits x M x N x 4 bytes; ask unit_gemm_f16_ws_bytes) are rejected with UNIT_E_ARG: pass a workspace to
 * unit_gemm_f16_ws instead.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two
 * streams, two threads) race, calls in stream order do not.  The first call on a device resolves the array's
 * address there; make it outside graph capture. */
int unit_gemm_f16_static(const void *a, const void *b, void *c, int32_t M, int32_t N, int32_t K, int32_t out_f16,
                         unit_stream_t stream);

/* _conv2d_NCHW16c_OHWI16o_impl(a, b, stride_h, stride_w, out_type)
 * (python/tensorizer/ops/gpu.py:8-53) on packed operands:
 *   a   f16 (N, C/16, H, W, 16)
 *   b   f16 (K/16, C/16, KH, KW, 16 in, 16 out)
 *   out f32 (N, K/16, OH, OW, 16)
 * Valid convolution: the descriptor's padding must be 0 and dilation 1, cb == 16 (the
 * reference operator has no padding argument; callers pre-pad). */
int unit_conv2d_nchw16c_f16f32(const unit_conv_desc *d, const void *a, const void *b, void *out,
                               unit_stream_t stream);

/* ------------------------------------------------------------------ layout / pre-pack */

/* layout_transform NCHW -> NCHW{cb}c (apps/cpu/relay/result.log:7,6807-6808; in-op form
 * python/tensorizer/ops/gpu.py:26-28): dst[n][ci][h][w][c] = src[n][cb*ci+c][h][w], zero for
 * cb*ci+c >= C.  elem_size is the element width in bytes (1, 2 or 4). */
int unit_pack_nchwc(const void *src, void *dst, int32_t N, int32_t C, int32_t H, int32_t W,
                    int32_t cb, int32_t elem_size, unit_stream_t stream);

/* layout_transform NCHW{cb}c -> NCHW (apps/cpu/relay/result.log:25), keeping the first C
 * channels of the ceil(C/cb) blocks. */
int unit_unpack_nchwc(const void *src, void *dst, int32_t N, int32_t C, int32_t H, int32_t W,
                      int32_t cb, int32_t elem_size, unit_stream_t stream);

/* int8 conv weight pre-pack OIHW -> (ceil(O/16), ceil(I/cb), KH, KW, cb/4, 16, 4): the
 * transpose/reshape chain of apps/cpu/relay/result.log:8-13 (cb = 16) and :6809-6815
 * (cb = 4, input channels zero-padded);  dst[ko][ci][kh][kw][e][kb][i] =
 * src[16ko+kb][cb*ci+4e+i][kh][kw], zero outside O x I. */
int unit_prepack_conv_weight_s8(const void *src, void *dst, int32_t O, int32_t I, int32_t KH,
                                int32_t KW, int32_t cb, unit_stream_t stream);

/* int8 dense weight pre-pack (N, K) -> (N/128, K/4, 128, 4) (placeholder shape at
 * apps/cpu/kernel/int8-gemm.py:14; 16x4 analogue poc/vnni/vnni_dense.py:10-11). */
int unit_prepack_dense_weight_s8(const void *src, void *dst, int32_t N, int32_t K,
                                 unit_stream_t stream);

/* fp16 conv weight pack OIHW -> (O/16, I/16, KH, KW, 16 in, 16 out)
 * (python/tensorizer/ops/gpu.py:29-31).  O % 16 == 0, I % 16 == 0. */
int unit_prepack_conv_weight_f16(const void *src, void *dst, int32_t O, int32_t I, int32_t KH,
                                 int32_t KW, unit_stream_t stream);

/* The same GEMM with b prepared once: bt f16 (N, K) = b^T, K-contiguous like a, so that both
 * operand tiles go from global memory straight into LDS (no register round trip, no transposition
 * while staging).  The reference's analogue is the one-time re-layout of b in
 * apps/gpu/gemm-pack.py:9,17 (b pre-packed as (N/32, K/32, 32, 32) for its wmma loads).
 * unit_gemm_f16_prepare_b writes bt (N * K halves, caller-owned) from b (K, N); K % 8 == 0.
 * unit_gemm_f16_prepared: c (M, N) = a (M, K) . bt^T, same results as unit_gemm_f16 (the same
 * products summed in the same order); K % 8 == 0, N % 4 == 0. */
int unit_gemm_f16_prepare_b(const void *b, void *bt, int32_t K, int32_t N, unit_stream_t stream);
/* The same bt from a b that is already in the reference's packed form (apps/gpu/gemm-pack.py:9,17):
 * bp f16 (N/32, K/32, 32, 32), bp[y/32][k/32][k%32][y%32] = b[k][y]; K % 32 == 0, N % 32 == 0. */
int unit_gemm_f16_prepare_b_packed32(const void *bp, void *bt, int32_t K, int32_t N, unit_stream_t stream);
int unit_gemm_f16_prepared(const void *a, const void *bt, void *c, int32_t M, int32_t N, int32_t K,
                           int32_t out_f16, unit_stream_t stream);

/* Alignment: every tensor pointer passed to a convolution, dense, GEMM or prepare entry point
 * must be 16-byte aligned (the kernels use 16-byte vector accesses); a misaligned one is
 * rejected with UNIT_E_ARG.  Framework allocations (256 bytes and up) satisfy this; a view that
 * starts inside an allocation may not. */

/* ------------------------------------------------------------------ prepared weights */

/* Convolution weights re-ordered once into the MFMA fragment order of the kernels, with the
 * per-channel term of the u8 shift (128 * sum of the channel's weights) precomputed.  The
 * reference's compiled graphs hold the same two pieces as constant sub-graphs next to the
 * convolution: the weight layout chain (apps/cpu/relay/result.log:8-13) and sum(w) over
 * (I, KH, KW) (result.log:15-16).  A convolution on prepared weights reads a lane's fragment with
 * one 16-byte load and accumulates no weight sums in its reduction loop.
 *
 * weight: the blocked layout the convolutions above take, K a multiple of 16 and C of cb:
 *   elem_bytes 1: s8 (K/16, C/cb, KH, KW, cb/4, 16, 4), cb = 16, or cb = 4 with KW <= 8 (the stem);
 *   elem_bytes 2: f16 (K/16, C/16, KH, KW, 16 in, 16 out), cb = 16.
 * prepared: unit_conv2d_prepared_weight_bytes() bytes, 16-byte aligned, owned by the caller:
 *   [ceil(K/32)][k-step][64 lanes][16 bytes] (+ int32 addend[ceil(K/32) * 32] for int8); it depends
 *   on the weight only, not on the image size, stride or padding. */
int unit_conv2d_prepared_weight_bytes(int32_t K, int32_t C, int32_t KH, int32_t KW, int32_t cb,
                                      int32_t elem_bytes, size_t *bytes);
int unit_conv2d_prepare_weight(int32_t K, int32_t C, int32_t KH, int32_t KW, int32_t cb, int32_t elem_bytes,
                               const void *weight, void *prepared, unit_stream_t stream);

/* The convolutions above on prepared weights; same results (int8: bit for bit; fp16: the same
 * products summed in the same order).  d->cb == 16 with int8 windows of at most 31 positions, or
 * (int8 only) d->cb == 4 with KW <= 8, KH <= 31 and no dilation along W.  Replace the same reference calls as unit_conv2d_nchwc_u8s8s32
 * (apps/cpu/kernel/conv2d.py:50-51), unit_conv2d_nchwc_s8s8s32_fused (result.log:3-26) and
 * unit_conv2d_nchw16c_f16f32 (python/tensorizer/ops/gpu.py:8-53). */
int unit_conv2d_nchwc_u8s8s32_prepared(const unit_conv_desc *d, const void *data, const void *prepared,
                                       void *out, unit_stream_t stream);
int unit_conv2d_nchwc_s8s8s32_fused_prepared(const unit_conv_desc *d, const void *data, const void *prepared,
                                             const int32_t *bias, int32_t scale, void *out,
                                             unit_stream_t stream);
int unit_conv2d_nchw16c_f16f32_prepared(const unit_conv_desc *d, const void *a, const void *prepared,
                                        void *out, unit_stream_t stream);

/* unit_conv2d_nchwc_s8s8s32_fused_prepared with the graph's closing layout_transform NCHW16c -> NCHW
 * (apps/cpu/relay/result.log:25, Op "fused_layout_transform" of :36) folded into the store:
 * out is (N, out_channels, OH, OW) int32, d->K - 16 < out_channels <= d->K (channels the caller
 * padded up to a multiple of 16 are not written). */
int unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw(const unit_conv_desc *d, const void *data, const void *prepared,
                                                  const int32_t *bias, int32_t scale, void *out,
                                                  int32_t out_channels, unit_stream_t stream);

/* u8 x s8 convolution on prepared weights with the output requantised to u8 in the blocked
 * layout the next convolution reads, (N, K/16, OH, OW, 16) u8:
 *   q = clamp(((conv_u8(data, w)[k] + bias[k]) * scale + 2^(shift-1)) >> shift, 0, 255)
 * (sum and bias in int32, product and shift in 64 bits, 1 <= shift <= 62; the lower clamp is the
 * ReLU).  bias: K int32 values or NULL.  Four times less output traffic than the int32 forms.
 * No counterpart in the reference's files: its printed graphs stop at the int32
 * subtract / add / multiply (apps/cpu/relay/result.log:15-24); this is the integer requantisation
 * that follows it in a quantised network, defined here and by the oracle of the same name. */
int unit_conv2d_nchwc_u8s8u8_requant_prepared(const unit_conv_desc *d, const void *data, const void *prepared,
                                              const int32_t *bias, int32_t scale, int32_t shift, void *out,
                                              unit_stream_t stream);

/* ------------------------------------------------------------------ diagnostics */

/* One v_mfma_i32_32x32x32_i8 / v_mfma_f32_32x32x16_f16 on a single wavefront, operands and
 * result in plain row-major form:  a (32, 32) s8 | f16 (32, 16);  b (32 cols, 32) s8 |
 * (32 cols, 16) f16 given K-contiguous per column;  c (32, 32) i32 | f32 = a . b^T.
 * The counterpart of poc/vnni/poc.cc:17-38 (instruction-semantics check). */
int unit_mfma_tile_i8(const void *a, const void *b, void *c, unit_stream_t stream);
int unit_mfma_tile_f16(const void *a, const void *b, void *c, unit_stream_t stream);

/* Register-only MFMA throughput probe, the counterpart of the reference's vpdpbusd peak
 * micro-benchmark (poc/vnni/micro.cc:16-51): `blocks` workgroups of 4 wavefronts each issue
 * 4 * iters MFMAs per wavefront (int8 32x32x32 when f16 == 0, else fp16 32x32x16) on 4
 * independent accumulator chains with no memory traffic.  Operations issued =
 * blocks * 4 * 4 * iters * 65536 (int8) or * 32768 (fp16); the caller times the launch.
 * `f16` bit 1 (values 2, 3) selects operands with random bit patterns that change from one
 * instruction to the next instead of constant ones: the chip's clocks follow its power draw, and
 * the rate it sustains depends on how many operand bits toggle.  For int8 those operands are
 * uniform random bytes, i.e. the distribution of the 4096^3 int8 benchmark; f16 == 5 draws the
 * fp16 operands like the fp16 benchmark does (x ~ N(0,1)/64, y ~ N(0,1)) instead of hashed bits.
 * `sink` is a 4-byte device scratch word. */
int unit_mfma_peak(int32_t f16, int32_t blocks, int32_t iters, void *sink, unit_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* UNIT_AMD_H */
