"""Parity of the int8 HIP path (through the C ABI) against the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

import unit_amd as U
from unit_amd import rng

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def test_mfma_tile_i8_lane_layout(dev):
    """One v_mfma_i32_32x32x32_i8 against the integer matrix product: pins the operand / result
    lane mapping every kernel relies on (the counterpart of the vpdpbusd known-answer program)."""
    import ctypes
    from unit_amd import _lib
    a = rng.uniform_s8((32, 32), 11)
    b = rng.uniform_s8((32, 32), 12)
    ta, tb = _t(a, dev), _t(b, dev)
    tc = torch.zeros((32, 32), dtype=torch.int32, device=dev)
    _lib.check(_lib.load().unit_mfma_tile_i8(ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), None))
    torch.cuda.synchronize()
    ref = a.astype(np.int64) @ b.astype(np.int64).T
    assert np.array_equal(tc.cpu().numpy(), ref.astype(np.int32))


DENSE_CASES = [
    # M, N, K
    (1, 128, 16),          # the reference's M=1 dense (cpu-shapes.log:367) in miniature
    (1, 1024, 512),        # resnet18 classifier: (1, 512) x (8, 128, 128, 4)
    (128, 3072, 768),      # apps/cpu/kernel/int8-gemm.py:9
    (37, 256, 80),         # ragged M, K not a multiple of the stage
    (300, 384, 272),
    (4096, 2048, 256),     # large-tile variant (128 workgroups of 256x256)
    (2100, 4096, 144),     # large tiles with a ragged M edge and a K tail
]


@pytest.mark.parametrize("M,N,K", DENSE_CASES)
@pytest.mark.parametrize("packed", [True, False])
def test_dense_bit_exact(dev, oracle, M, N, K, packed):
    a = rng.uniform_u8((M, K), 100 + M)
    w = rng.uniform_s8((N, K), 200 + N)
    wp = oracle.prepack_dense_weight(w)
    ref = oracle.c_dense(a, wp)
    if M * N * K <= 1 << 24:
        assert np.array_equal(ref, oracle.dense_logical(a, w))
    out = U.dense_dotprod(_t(a, dev), _t(wp if packed else w, dev))
    torch.cuda.synchronize()
    assert out.dtype == torch.int32 and tuple(out.shape) == (M, N)
    assert np.array_equal(out.cpu().numpy(), ref), U.last_variant()


@pytest.mark.parametrize("M,N,K,kernel", [(1, 4, 64, "dma_x128_y128_k64_w2x2_r4_s1"), (5, 12, 128, "dma_x128_y128"),
                                          (130, 132, 192, "dma_x128_y128"), (1000, 520, 320, "dma_x128_y128"),
                                          (4096, 4096, 192, "i8denserm_x256"), (4096, 3840, 256, "i8densedma_x256_y256"),
                                          (2800, 4000, 384, "i8densedma_x256_y256")])
def test_dense_row_major_direct_to_lds_edges(dev, oracle, M, N, K, kernel):
    """Row-major weights with a reduction of whole 64-byte stages run the 128 x 128 all-direct tiles (in-kernel weight
    sums): one stage only, a single row, N of one 4-column group, ragged tile edges; shapes that 256 x 256 tiles fill
    better run those on the same pipeline when the reduction is a whole number of 128-byte stages (the four waves that
    share a weight fragment divide the weight sums between them; ragged M and N edges, an odd number of stages), else
    stay on the register pipeline.  The same on a prepared weight."""
    a = rng.uniform_u8((M, K), 900 + M)
    w = rng.uniform_s8((N, K), 901 + N)
    ref = oracle.dense_logical(a, w) if M * N * K <= 1 << 28 else None
    ta, tw = _t(a, dev), _t(w, dev)
    out = U.dense(ta, tw)
    assert kernel in U.last_variant(), U.last_variant()
    if ref is None:
        ref = (ta.double() @ tw.double().T).cpu().numpy().astype(np.int64)
    assert np.array_equal(out.cpu().numpy(), ref), U.last_variant()
    assert torch.equal(U.dense(ta, U.prepare_dense_weight(tw)), out), U.last_variant()


@pytest.mark.parametrize("M,N,K", [(300, 384, 272), (37, 256, 16), (512, 640, 400), (1, 128, 48)])
def test_dense_packed_weights_direct_to_registers(dev, oracle, monkeypatch, M, N, K):
    """The kernel variant that reads the pre-packed weight straight into MFMA fragments, forced on
    ragged shapes: M and N tile edges, a K tail of 16 .. 112 bytes, one k-step."""
    monkeypatch.setenv("UNIT_AMD_DENSE_VARIANT", "13")
    a = rng.uniform_u8((M, K), 300 + M)
    wp = oracle.prepack_dense_weight(rng.uniform_s8((N, K), 400 + N))
    out = U.dense_dotprod(_t(a, dev), _t(wp, dev))
    torch.cuda.synchronize()
    assert "direct" in U.last_variant()
    assert np.array_equal(out.cpu().numpy(), oracle.c_dense(a, wp)), U.last_variant()


@pytest.mark.parametrize("M,N,K", [(128, 768, 3072), (50, 260, 1040), (1, 128, 8192)])
def test_dense_k_splits_bit_exact(dev, oracle, M, N, K):
    """Few output tiles: the reduction is shared between workgroups (int32 atomics, exact in any order); the output
    buffer's previous contents must not leak into the sums."""
    a = rng.uniform_u8((M, K), 500 + M)
    w = rng.uniform_s8((N, K), 600 + N)
    ref = oracle.dense_logical(a, w) if N % 128 else oracle.c_dense(a, oracle.prepack_dense_weight(w))
    out = U.dense(_t(a, dev), _t(w, dev))
    assert int(U.last_variant().rsplit("_s", 1)[1]) > 1, U.last_variant()
    assert np.array_equal(out.cpu().numpy(), ref)
    from unit_amd import _lib
    garbage = torch.full((M, N), 12345, dtype=torch.int32, device=dev)
    ta, tw = _t(a, dev), _t(w, dev)
    _lib.check(_lib.load().unit_dense_u8s8s32(ta.data_ptr(), tw.data_ptr(), garbage.data_ptr(), M, N, K,
                                              torch.cuda.current_stream().cuda_stream))
    assert np.array_equal(garbage.cpu().numpy(), ref)


def test_dense_largest_output(dev, oracle):
    """An output just below the 2^31-byte limit (23168^2 int32 = 2.147 GB): 32-bit offsets must not wrap."""
    M = N = 23168
    K = 32
    assert M * N * 4 < 2 ** 31 <= (M + 128) * N * 4
    a = rng.uniform_u8((M, K), 71)
    w = rng.uniform_s8((N, K), 72)
    out = U.dense(_t(a, dev), _t(w, dev))
    torch.cuda.synchronize()
    for rows in (slice(0, 64), slice(M // 2 - 32, M // 2 + 32), slice(M - 64, M)):
        ref = a[rows].astype(np.int64) @ w.astype(np.int64).T
        assert np.array_equal(out[rows].cpu().numpy().astype(np.int64), ref), U.last_variant()
    del out
    torch.cuda.empty_cache()


def test_dense_extremes(dev, oracle):
    """255 x -128 everywhere: the largest negative accumulation (K * -32640), and 255 x 127."""
    M, N, K = 64, 128, 4096
    a = np.full((M, K), 255, dtype=np.uint8)
    for val in (-128, 127):
        w = np.full((N, K), val, dtype=np.int8)
        out = U.dense(_t(a, dev), _t(w, dev)).cpu().numpy()
        assert (out == 255 * val * K).all()
    # zeros stay zero (the u8 -> s8 shift and its correction cancel)
    out = U.dense(_t(np.zeros((M, K), np.uint8), dev), _t(rng.uniform_s8((N, K), 5), dev)).cpu().numpy()
    assert (out == 0).all()


CONV_CASES = [
    # N, C, H, W, K, kernel, stride, pad, dilation
    (1, 64, 56, 56, 64, 3, 1, 1, 1),       # the single-convolution benchmark configuration
    (2, 32, 9, 7, 32, 3, 1, 1, 1),         # tiny, ragged pixel count
    (1, 16, 8, 8, 48, 1, 2, 0, 1),         # 1x1 stride 2, K not a multiple of 32
    (3, 64, 14, 14, 128, 1, 1, 0, 1),      # 1x1 = GEMM
    (1, 128, 28, 28, 128, 3, 1, 1, 1),
    (1, 64, 56, 56, 128, 3, 2, 1, 1),
    (1, 256, 14, 14, 512, 3, 2, 1, 1),
    (1, 512, 7, 7, 512, 3, 1, 1, 1),
    (1, 4, 32, 32, 64, 7, 2, 3, 1),        # NCHW4c stem, small
    (1, 4, 224, 224, 64, 7, 2, 3, 1),      # NCHW4c stem, full size
    (2, 8, 11, 13, 16, 3, 1, (0, 1, 2, 1), 1),   # cb = 4 with two channel blocks, asymmetric pad
    (2, 16, 12, 12, 32, 3, 1, 2, 2),       # dilation 2
    (1, 48, 10, 10, 80, 5, (2, 1), (2, 0), 1),   # anisotropic stride / pad, 5x5
    (32, 64, 56, 56, 64, 1, 1, 0, 1),      # batch 32: 64-channel tile, many workgroups
    (32, 256, 14, 14, 256, 3, 1, 1, 1),    # batch 32: 256-channel tile
    (32, 128, 28, 28, 128, 3, 1, 1, 1),    # batch 32: 128-channel tile
    (8, 512, 7, 7, 2048, 1, 1, 0, 1),
    (1, 16, 5, 5, 32, 3, 1, 3, 1),         # padding as wide as the window: border windows lie outside altogether
    (2, 32, 2, 3, 32, 3, 1, 1, 1),         # image smaller than the window: cut on both sides at once
    (1, 16, 3, 3, 16, 5, 1, 2, 1),         # 5x5 on 3x3: every window loses rows and columns at both ends
    (2, 32, 6, 9, 32, 3, 2, (2, 0, 1, 3), 1),   # stride 2, four different pads
]


@pytest.mark.parametrize("N,C,H,W,K,ks,stride,pad,dil", CONV_CASES)
def test_conv2d_bit_exact(dev, oracle, N, C, H, W, K, ks, stride, pad, dil):
    cb = 16 if C % 16 == 0 else 4
    data = rng.uniform_u8((N, C // cb, H, W, cb), 7 * C + H)
    wt = rng.uniform_s8((K // 16, C // cb, ks, ks, cb // 4, 16, 4), 3 * K + ks)
    ref = oracle.c_conv2d_nchwc(data, wt, stride, pad, dil)
    out = U.conv2d_NCHWc_int8(_t(data, dev), _t(wt, dev), stride, pad, dil, "int32", f"NCHW{cb}c", "NCHW16c")
    torch.cuda.synchronize()
    assert tuple(out.shape) == ref.shape
    assert np.array_equal(out.cpu().numpy(), ref), U.last_variant()


VARIANT_CASES = [
    # N, C, H, W, K, kernel, stride, pad: reductions of 1 .. 12 pipeline stages, ragged tiles
    (2, 80, 9, 11, 96, 3, 1, 1),    # 720 reduction bytes: the last stage is partly padding
    (1, 32, 5, 5, 16, 1, 1, 0),     # one stage: k-groups beyond the first have nothing to do
    (1, 48, 6, 6, 32, 3, 1, 1),     # 432 bytes: 4 or 7 stages, shared unevenly by 2 or 4 k-groups
    (3, 256, 7, 7, 160, 3, 2, 1),   # 2304 bytes: a long reduction over few pixels
    (1, 4, 16, 16, 32, 7, 2, 3),    # NCHW4c
]


@pytest.mark.parametrize("N,C,H,W,K,ks,stride,pad", VARIANT_CASES)
def test_conv2d_every_variant(dev, oracle, monkeypatch, N, C, H, W, K, ks, stride, pad):
    """Every tile variant the planner can pick (and k-splits of it) gives the oracle's result."""
    from unit_amd import _lib
    cb = 16 if C % 16 == 0 else 4
    data = rng.uniform_u8((N, C // cb, H, W, cb), 11 * C + H)
    wt = rng.uniform_s8((K // 16, C // cb, ks, ks, cb // 4, 16, 4), 5 * K + ks)
    ref = oracle.c_conv2d_nchwc(data, wt, stride, pad, 1)
    d, w = _t(data, dev), _t(wt, dev)
    count = _lib.load().unit_conv_variant_count()
    assert count >= 40
    ran = set()
    for v in range(1, count + 1):
        if _lib.load().unit_conv_variant_is_direct(v - 1) == 2:
            continue  # LDS-shared variants exist for prepared weights only: the id runs the heuristic's choice here
        for splits in (1, 3):
            monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
            monkeypatch.setenv("UNIT_AMD_CONV_SPLITK", str(splits))
            try:
                out = U.conv2d_NCHWc_int8(d, w, stride, pad, 1, "int32", f"NCHW{cb}c", "NCHW16c")
            except ValueError as e:  # a variant may only be refused for its LDS budget or its layout
                assert "LDS" in str(e) or "not available" in str(e), (v, str(e))
                continue
            torch.cuda.synchronize()
            ran.add((v, U.last_variant()))
            assert np.array_equal(out.cpu().numpy(), ref), (v, U.last_variant())
    # the override really switched kernels: as many kernel names as variants that ran
    assert len({name for _, name in ran}) >= len({v for v, _ in ran}) >= 46


FUSED_CASES = [
    # N, C, H, W, K, kernel, stride, pad, with bias
    (1, 1024, 16, 16, 2048, 1, 1, 0, True),     # apps/cpu/relay/result.log:3-26
    (1, 3, 224, 224, 64, 7, 2, 0, True),        # result.log:6803-6828 (channels padded to 4: NCHW4c)
    (2, 64, 14, 14, 96, 3, 1, 1, True),         # zero padding in the signed domain
    (3, 48, 9, 11, 80, 3, 2, (1, 0, 2, 1), False),
    (32, 256, 14, 14, 256, 3, 1, 1, True),      # ResNet-50 batch 32 layer
    (1, 16, 20, 20, 32, 7, 1, 3, True),         # 49-position window on NCHW16c: staged kernel
    (2, 32, 5, 5, 16, 1, 1, 0, False),          # one k-step
]


@pytest.mark.parametrize("N,C,H,W,K,ks,stride,pad,with_bias", FUSED_CASES)
def test_conv2d_fused_bit_exact(dev, oracle, N, C, H, W, K, ks, stride, pad, with_bias):
    """(conv(x_s8 + 128, w) - 128 sum(w) + bias) * scale of the reference's quantized graphs."""
    cb = 16 if C % 16 == 0 else 4
    x = oracle.pack_nchwc(rng.uniform_s8((N, C, H, W), 13 * C + H), cb)
    wt = rng.uniform_s8((K // 16, x.shape[1], ks, ks, cb // 4, 16, 4), 7 * K + ks)
    bias = (rng.uniform_s8((K,), 5).astype(np.int32) * 4099) if with_bias else None
    ref = oracle.conv2d_nchwc_int8_fused(x, wt, bias, 11, stride, pad, 1, conv=oracle.c_conv2d_nchwc)
    out = U.conv2d_NCHWc_int8_fused(_t(x, dev), _t(wt, dev), _t(bias, dev) if with_bias else None, 11, stride, pad, 1,
                                    "int32", f"NCHW{cb}c", "NCHW16c")
    torch.cuda.synchronize()
    assert tuple(out.shape) == ref.shape
    assert np.array_equal(out.cpu().numpy(), ref), U.last_variant()


def test_conv2d_fused_every_direct_variant(dev, oracle, monkeypatch):
    from unit_amd import _lib
    N, C, H, W, K, ks = 2, 80, 9, 11, 96, 3
    x = rng.uniform_s8((N, C // 16, H, W, 16), 3)
    wt = rng.uniform_s8((K // 16, C // 16, ks, ks, 4, 16, 4), 4)
    bias = rng.uniform_s8((K,), 5).astype(np.int32) * 77
    ref = oracle.conv2d_nchwc_int8_fused(x, wt, bias, -3, 1, 1, 1, conv=oracle.c_conv2d_nchwc)
    tx, tw, tb = _t(x, dev), _t(wt, dev), _t(bias, dev)
    names = set()
    for v in range(1, _lib.load().unit_conv_variant_count() + 1):
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        out = U.conv2d_NCHWc_int8_fused(tx, tw, tb, -3, 1, 1)
        torch.cuda.synchronize()
        names.add(U.last_variant())
        assert np.array_equal(out.cpu().numpy(), ref), (v, U.last_variant())
    assert len(names) >= 15 and all(n.startswith("s8direct") for n in names)


CONV3D_CASES = [
    # C, D, H, W, K, kernel, stride: apps/cpu/kernel/conv3d.py:13-25 (d = 16 there; depth cut where the oracle would take minutes)
    (256, 16, 16, 16, 256, 3, 1),
    (512, 16, 9, 9, 512, 3, 1),
    (128, 6, 30, 30, 128, 3, 1),
    (64, 16, 56, 56, 128, 1, 2),
    (64, 5, 58, 58, 64, 3, 1),
    (256, 16, 16, 16, 512, 3, 2),
    (256, 16, 14, 14, 512, 1, 2),
    (16, 4, 7, 9, 32, 3, 1),      # 27 taps: odd, the last k-step is half padding; ragged pixel count
    (48, 3, 5, 5, 16, (1, 3, 2), 1),
    (4, 9, 38, 38, 64, 7, 2),     # conv3d.py:22 (230 x 230 there), 3 -> 4 channels: 4-channel blocks
    (8, 5, 9, 11, 32, (2, 3, 8), 1),   # two 4-channel blocks, rows of 8 taps
    (12, 4, 6, 7, 48, (3, 1, 5), 2),
]


@pytest.mark.parametrize("C,D,H,W,K,ks,stride", CONV3D_CASES)
def test_conv3d_bit_exact(dev, oracle, C, D, H, W, K, ks, stride):
    kd, kh, kw = (ks,) * 3 if isinstance(ks, int) else ks
    cb = 4 if C % 16 else 16     # the channel block rule of apps/cpu/kernel/conv3d.py:39-56
    x = rng.uniform_s8((1, C // cb, D, H, W, cb), 17 * C + H)
    wt = rng.uniform_s8((K // 16, C // cb, kd, kh, kw, cb // 4, 16, 4), 19 * K + kd)
    ref = oracle.conv3d_ncdhwc_int8(x, wt, stride)
    out = U.conv3d_NCDHWc_int8(_t(x, dev), _t(wt, dev), stride)
    torch.cuda.synchronize()
    assert tuple(out.shape) == ref.shape
    assert ("_c4_" in U.last_variant()) == (cb == 4)
    assert np.array_equal(out.cpu().numpy(), ref), U.last_variant()


def test_conv3d_every_direct_variant(dev, oracle, monkeypatch):
    from unit_amd import _lib
    x = rng.uniform_s8((2, 3, 5, 7, 9, 16), 23)
    wt = rng.uniform_s8((5, 3, 3, 3, 3, 4, 16, 4), 29)
    ref = oracle.conv3d_ncdhwc_int8(x, wt, 1)
    tx, tw = _t(x, dev), _t(wt, dev)
    for v in range(1, _lib.load().unit_conv_variant_count() + 1):
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        out = U.conv3d_NCDHWc_int8(tx, tw, 1)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), ref), (v, U.last_variant())


def test_conv3d_c4_every_direct_variant(dev, oracle, monkeypatch):
    from unit_amd import _lib
    x = rng.uniform_s8((2, 2, 6, 8, 13, 4), 31)
    wt = rng.uniform_s8((3, 2, 3, 2, 5, 1, 16, 4), 37)
    ref = oracle.conv3d_ncdhwc_int8(x, wt, 1)
    tx, tw = _t(x, dev), _t(wt, dev)
    names = set()
    for v in range(1, _lib.load().unit_conv_variant_count() + 1):
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        out = U.conv3d_NCDHWc_int8(tx, tw, 1)
        torch.cuda.synchronize()
        names.add(U.last_variant())
        assert np.array_equal(out.cpu().numpy(), ref), (v, U.last_variant())
    assert len(names) >= 15 and all(n.startswith("s8direct_c4") for n in names), names


def test_conv2d_largest_output(dev, oracle):
    """An output just below the 2^31-byte limit (100352 pixels x 5344 channels x 4 bytes = 2.145 GB): 32-bit
    offsets in the write-back must not wrap.  Checked plane by plane against the oracle run on slices of the
    weight (first, middle and last 16-channel blocks)."""
    N, C, H, W, K = 32, 16, 56, 56, 5344
    assert N * H * W * K * 4 < 2 ** 31 <= N * H * W * (K + 16) * 4
    data = rng.uniform_u8((N, 1, H, W, 16), 81)
    wt = rng.uniform_s8((K // 16, 1, 1, 1, 4, 16, 4), 82)
    out = U.conv2d_NCHWc_int8(_t(data, dev), _t(wt, dev), 1, 0)
    torch.cuda.synchronize()
    name = U.last_variant()
    for ko in (0, 1, K // 32, K // 16 - 2, K // 16 - 1):
        ref = oracle.c_conv2d_nchwc(data, wt[ko:ko + 1], 1, 0, 1)
        assert np.array_equal(out[:, ko:ko + 1].cpu().numpy(), ref), (ko, name)
    del out
    torch.cuda.empty_cache()


def test_conv2d_zero_padding_value(dev, oracle):
    """Padded pixels are u8 zeros: with all-255 data and all-ones weights every output equals
    255 * (number of in-image taps) * C, which differs between border and interior."""
    C, H, K = 16, 6, 16
    data = np.full((1, 1, H, H, 16), 255, dtype=np.uint8)
    wt = np.ones((1, 1, 3, 3, 4, 16, 4), dtype=np.int8)
    out = U.conv2d_NCHWc_int8(_t(data, dev), _t(wt, dev), 1, 1).cpu().numpy()
    assert out[0, 0, 0, 0, 0] == 255 * 4 * C and out[0, 0, 2, 2, 0] == 255 * 9 * C
    assert np.array_equal(out, oracle.conv2d_nchwc_int8(data, wt, 1, 1))


def _golden(pattern):
    import glob
    import os
    return sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", pattern)))


@pytest.mark.parametrize("path", _golden("conv_*.npz"))
def test_conv2d_golden_fixtures(dev, path):
    g = np.load(path)
    st, pad, dil, cb = (int(x) for x in g["params"])
    out = U.conv2d_NCHWc_int8(_t(g["data"], dev), _t(g["weight"], dev), st, pad, dil, "int32", f"NCHW{cb}c")
    assert np.array_equal(out.cpu().numpy(), g["out"])


@pytest.mark.parametrize("path", _golden("dense_*.npz"))
def test_dense_golden_fixtures(dev, path):
    g = np.load(path)
    assert np.array_equal(U.dense_dotprod(_t(g["a"], dev), _t(g["wp"], dev)).cpu().numpy(), g["out"])
    assert np.array_equal(U.dense(_t(g["a"], dev), _t(g["w"], dev)).cpu().numpy(), g["out"])
    assert np.array_equal(U.prepack_dense_weight(_t(g["w"], dev)).cpu().numpy(), g["wp"])


def test_full_size_properties(dev):
    """Benchmark-size checks that need no CPU reference: 4096^3 int8 GEMM and a batch-32 ResNet-50
    layer through size-independent properties (linearity in the weights, the packed and un-packed
    weight paths agree, all-ones weights give per-row activation sums)."""
    M = N = K = 4096
    a = _t(rng.uniform_u8((M, K), 41), dev)
    w1 = rng.uniform_s8((N, K), 42) // 2
    w2 = rng.uniform_s8((N, K), 43) // 2
    c1 = U.dense(a, _t(w1.astype(np.int8), dev))
    c2 = U.dense(a, _t(w2.astype(np.int8), dev))
    c12 = U.dense(a, _t((w1 + w2).astype(np.int8), dev))
    assert torch.equal(c12, c1 + c2)
    assert torch.equal(U.dense_dotprod(a, U.prepack_dense_weight(_t(w1.astype(np.int8), dev))), c1)
    ones = torch.ones((128, K), dtype=torch.int8, device=dev)
    rowsum = a.to(torch.int32).sum(dim=1, dtype=torch.int32)
    assert torch.equal(U.dense(a, ones), rowsum[:, None].expand(M, 128))
    # batch-32 3x3 256 -> 256 @ 14: every image of a batch of identical images gives the same output,
    # and equals the batch-1 result
    d1 = rng.uniform_u8((1, 16, 14, 14, 16), 44)
    wt = _t(rng.uniform_s8((16, 16, 3, 3, 4, 16, 4), 45), dev)
    o1 = U.conv2d_NCHWc_int8(_t(d1, dev), wt, 1, 1)
    o32 = U.conv2d_NCHWc_int8(_t(np.repeat(d1, 32, axis=0), dev), wt, 1, 1)
    assert torch.equal(o32, o1.expand(32, -1, -1, -1, -1))


@pytest.mark.parametrize("M,N,K,kernel", [(512, 8192, 256, "prep_dma_x128_y128"), (4096, 4096, 128, "prep_dma_x256_y256"),
                                          (2000, 4100, 384, "prep_dma_x256_y256"), (64, 128, 128, "prep_dma_x128_y128"),
                                          (128, 768, 3072, "prep_dma_x128_y128_k64_w2x2_r4_s12"),
                                          (300, 4096, 144, "i8denserm"), (4096, 4096, 192, "i8denserm")])
def test_dense_on_prepared_weight(dev, oracle, M, N, K, kernel):
    """Weight sums folded once (unit_dense_prepare_weight): both operands go global -> LDS directly, on 256 x 256
    tiles (whole 128-byte stages) where those fill the chip, else on 128 x 128 tiles (whole 64-byte stages), with
    k-splits when the tiles are few -- the sums are then added by one split only; ragged M / N included.  The other
    shapes fall back to the plain entry.  Bit-exact against a . W^T either way."""
    a = rng.uniform_u8((M, K), 70 + M)
    w = rng.uniform_s8((N, K), 71 + N)
    p = U.prepare_dense_weight(_t(w, dev))
    assert np.array_equal(p.wsum.cpu().numpy(), w.astype(np.int64).sum(axis=1))
    out = torch.full((M, N), 777, dtype=torch.int32, device=dev)  # k-splits must not add onto what was there
    from unit_amd import _lib
    ta = _t(a, dev)
    _lib.check(_lib.load().unit_dense_u8s8s32_prepared(ta.data_ptr(), p.w.data_ptr(), p.wsum.data_ptr(), out.data_ptr(), M, N, K,
                                                       torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert kernel in U.last_variant(), U.last_variant()
    assert np.array_equal(out.cpu().numpy(), oracle.dense_logical(a, w)), U.last_variant()
    assert torch.equal(U.dense(ta, p), out)


def test_dense_on_prepared_weight_extremes(dev, oracle):
    """255 x -128 everywhere: the largest magnitudes the u8 shift and its correction see."""
    M, N, K = 4096, 2048, 512
    a = np.full((M, K), 255, np.uint8)
    w = np.full((N, K), -128, np.int8)
    w[::3] = 127
    out = U.dense(_t(a, dev), U.prepare_dense_weight(_t(w, dev)))
    torch.cuda.synchronize()
    assert "prep_dma" in U.last_variant()
    assert np.array_equal(out.cpu().numpy(), oracle.dense_logical(a, w))
