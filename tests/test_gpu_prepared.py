"""Convolutions on prepared (MFMA-fragment-ordered) weights, through the C ABI: the prepared buffer
against its index formula, and the results against the CPU oracle (int8: bit-exact; fp16: 1e-2
max-rel against float64, and bit for bit against the convolution on the reference's layout)."""
import numpy as np
import pytest
import torch

import unit_amd as U
from unit_amd import rng

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2
ZERO_BYTES = 16384  # zero region behind prepared int8 weights


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _fragments_i8(wt):
    """prepared[kb][s][lane][16] and addend[kb * 32 + c] from (K/16, C/16, KH, KW, 4, 16, 4) s8, by the index
    formula: lane -> channel kb * 32 + lane % 32, tap 2 s + lane / 32, byte 4 e + i -> input channel 4 e + i."""
    ko, cc, kh, kw = wt.shape[:4]
    K, ntaps = ko * 16, cc * kh * kw
    nsteps, kblocks = (ntaps + 1) // 2, (K + 31) // 32
    # w[k][tap][ci16]
    w = wt.reshape(ko, ntaps, 4, 16, 4).transpose(0, 3, 1, 2, 4).reshape(K, ntaps, 16)
    full = np.zeros((kblocks * 32, nsteps * 2, 16), np.int8)
    full[:K, :ntaps] = w
    frag = full.reshape(kblocks, 32, nsteps, 2, 16).transpose(0, 2, 3, 1, 4).reshape(kblocks, nsteps, 64, 16)
    addend = np.zeros(kblocks * 32, np.int32)
    addend[:K] = 128 * w.astype(np.int64).sum(axis=(1, 2))
    return frag, addend


def _fragments_f16(b):
    """prepared[kb][tap][lane][8 halves] from (K/16, C/16, KH, KW, 16 in, 16 out) f16: lane -> channel
    kb * 32 + lane % 32, input channels 8 (lane / 32) .. + 8."""
    ko, cc, kh, kw = b.shape[:4]
    K, ntaps = ko * 16, cc * kh * kw
    kblocks = (K + 31) // 32
    w = b.reshape(ko, ntaps, 16, 16).transpose(0, 3, 1, 2).reshape(K, ntaps, 16)  # [k][tap][ci]
    full = np.zeros((kblocks * 32, ntaps, 16), np.float16)
    full[:K] = w
    return full.reshape(kblocks, 32, ntaps, 2, 8).transpose(0, 2, 3, 1, 4).reshape(kblocks, ntaps, 64, 8)


@pytest.mark.parametrize("K,C,ks", [(64, 64, 3), (48, 16, 3), (16, 32, 1), (96, 80, (1, 3))])
def test_prepared_buffer_int8(dev, K, C, ks):
    kh, kw = (ks, ks) if isinstance(ks, int) else ks
    wt = rng.uniform_s8((K // 16, C // 16, kh, kw, 4, 16, 4), K + C)
    p = U.prepare_conv2d_weight(_t(wt, dev))
    torch.cuda.synchronize()
    frag, addend = _fragments_i8(wt)
    buf = p.buf.cpu().numpy()
    # fragments, the 128 * sum(w) addends, then 16 KiB of zeros (what the LDS-shared kernels fetch for padded taps)
    assert buf.size == frag.size + addend.size * 4 + ZERO_BYTES
    assert np.array_equal(buf[:frag.size].view(np.int8).reshape(frag.shape), frag)
    assert np.array_equal(buf[frag.size:buf.size - ZERO_BYTES].view(np.int32), addend)
    assert not buf[buf.size - ZERO_BYTES:].any()


@pytest.mark.parametrize("K,C,kh,kw", [(64, 4, 7, 7), (48, 8, 3, 3), (16, 4, 2, 8), (32, 12, 1, 5)])
def test_prepared_buffer_int8_c4(dev, K, C, kh, kw):
    """4-channel blocks: k-step = (channel block, kh), lane -> channel kb * 32 + lane % 32 and taps
    kw = 4 (lane / 32) .. + 3 (zeros for kw >= KW)."""
    cc = C // 4
    wt = rng.uniform_s8((K // 16, cc, kh, kw, 1, 16, 4), K + C)
    p = U.prepare_conv2d_weight(_t(wt, dev))
    torch.cuda.synchronize()
    kblocks, nsteps = (K + 31) // 32, cc * kh
    w = wt.reshape(K // 16, cc * kh, kw, 16, 4).transpose(0, 3, 1, 2, 4).reshape(K, nsteps, kw, 4)  # [k][ci*KH+kh][kw][ci4]
    full = np.zeros((kblocks * 32, nsteps, 8, 4), np.int8)
    full[:K, :, :kw] = w
    frag = full.reshape(kblocks, 32, nsteps, 2, 16).transpose(0, 2, 3, 1, 4).reshape(kblocks, nsteps, 64, 16)
    addend = np.zeros(kblocks * 32, np.int32)
    addend[:K] = 128 * w.astype(np.int64).sum(axis=(1, 2, 3))
    buf = p.buf.cpu().numpy()
    # fragments, the 128 * sum(w) addends, then 16 KiB of zeros (what the LDS-shared kernels fetch for padded taps)
    assert buf.size == frag.size + addend.size * 4 + ZERO_BYTES
    assert np.array_equal(buf[:frag.size].view(np.int8).reshape(frag.shape), frag)
    assert np.array_equal(buf[frag.size:buf.size - ZERO_BYTES].view(np.int32), addend)
    assert not buf[buf.size - ZERO_BYTES:].any()


@pytest.mark.parametrize("K,C,ks", [(64, 64, 3), (48, 16, 1), (16, 48, 2)])
def test_prepared_buffer_fp16(dev, K, C, ks):
    b = rng.normal_f16((K // 16, C // 16, ks, ks, 16, 16), K + C)
    p = U.prepare_conv2d_weight(_t(b, dev))
    torch.cuda.synchronize()
    frag = _fragments_f16(b)
    buf = p.buf.cpu().numpy()
    assert buf.size == frag.size * 2
    assert np.array_equal(buf.view(np.float16).reshape(frag.shape), frag)


CONV_CASES = [
    # N, C, H, W, K, kernel, stride, pad, dilation
    (1, 64, 56, 56, 64, 3, 1, 1, 1),       # the single-convolution benchmark configuration
    (2, 32, 9, 7, 32, 3, 1, 1, 1),         # tiny, ragged pixel count
    (1, 16, 8, 8, 48, 1, 2, 0, 1),         # one tap (half a k-step), K not a multiple of 32
    (1, 16, 9, 9, 48, 3, 1, 0, 1),         # 9 taps, no padding: the kernel without tap masks on an odd tap count
    (3, 64, 14, 14, 128, 1, 1, 0, 1),      # 1x1 = GEMM
    (1, 256, 14, 14, 512, 3, 2, 1, 1),
    (1, 512, 7, 7, 512, 3, 1, 1, 1),
    (2, 16, 12, 12, 32, 3, 1, 2, 2),       # dilation 2
    (1, 48, 10, 10, 80, 5, (2, 1), (2, 0), 1),   # anisotropic stride / pad, 5x5, 75 taps
    (32, 64, 56, 56, 256, 1, 1, 0, 1),     # ResNet-50 batch 32 layers
    (32, 256, 14, 14, 256, 3, 1, 1, 1),
    (8, 512, 7, 7, 2048, 1, 1, 0, 1),
    (1, 16, 5, 5, 32, 3, 1, 3, 1),         # padding as wide as the window: border windows lie outside altogether
    (2, 32, 2, 3, 32, 3, 1, 1, 1),         # image smaller than the window: cut on both sides at once
    (1, 16, 3, 3, 16, 5, 1, 2, 1),         # 5x5 on 3x3: every window loses rows and columns at both ends
    (2, 32, 6, 9, 32, 3, 2, (2, 0, 1, 3), 1),   # stride 2, four different pads
]


@pytest.mark.parametrize("N,C,H,W,K,ks,stride,pad,dil", CONV_CASES)
def test_conv2d_prepared_bit_exact(dev, oracle, N, C, H, W, K, ks, stride, pad, dil):
    data = rng.uniform_u8((N, C // 16, H, W, 16), 7 * C + H)
    wt = rng.uniform_s8((K // 16, C // 16, ks, ks, 4, 16, 4), 3 * K + ks)
    ref = oracle.c_conv2d_nchwc(data, wt, stride, pad, dil)
    p = U.prepare_conv2d_weight(_t(wt, dev))
    out = U.conv2d_NCHWc_int8(_t(data, dev), p, stride, pad, dil, "int32", "NCHW16c", "NCHW16c")
    torch.cuda.synchronize()
    assert "prep" in U.last_variant()
    assert tuple(out.shape) == ref.shape
    assert np.array_equal(out.cpu().numpy(), ref), U.last_variant()


C4_CASES = [
    # N, C (padded to 4s), H, W, K, (KH, KW), stride, pad, dilation
    (1, 4, 32, 32, 64, (7, 7), 2, 3, 1),          # the stem, small
    (1, 4, 224, 224, 64, (7, 7), 2, 3, 1),        # the stem, full size (apps/cpu/relay/result.log:6803-6828)
    (2, 8, 11, 13, 16, (3, 3), 1, (0, 1, 2, 1), 1),   # two channel blocks, asymmetric pad
    (3, 4, 9, 10, 48, (5, 8), (2, 1), (2, 3), 1),     # KW = 8: both halves full; K not a multiple of 32
    (1, 12, 7, 7, 32, (3, 1), 1, 0, (2, 1)),          # one tap per row, dilation along H, no padding
    (2, 4, 6, 5, 16, (1, 1), 1, 0, 1),                # 1x1: one k-step
    (32, 4, 224, 224, 64, (7, 7), 2, 3, 1),           # ResNet-50 batch 32 stem
]


@pytest.mark.parametrize("N,C,H,W,K,ks,stride,pad,dil", C4_CASES)
def test_conv2d_prepared_c4_bit_exact(dev, oracle, N, C, H, W, K, ks, stride, pad, dil):
    kh, kw = ks
    data = rng.uniform_u8((N, C // 4, H, W, 4), 7 * C + H)
    wt = rng.uniform_s8((K // 16, C // 4, kh, kw, 1, 16, 4), 3 * K + kh)
    if N == 32:   # the oracle takes its time on the full batch: check two images of it
        ref = oracle.c_conv2d_nchwc(data[[0, 31]], wt, stride, pad, dil)
    else:
        ref = oracle.c_conv2d_nchwc(data, wt, stride, pad, dil)
    p = U.prepare_conv2d_weight(_t(wt, dev))
    out = U.conv2d_NCHWc_int8(_t(data, dev), p, stride, pad, dil, "int32", "NCHW4c", "NCHW16c")
    torch.cuda.synchronize()
    assert U.last_variant().startswith("i8prep_c4")
    got = out.cpu().numpy()
    if N == 32:
        got = got[[0, 31]]
    assert got.shape == ref.shape
    assert np.array_equal(got, ref), U.last_variant()
    # fused signed form on the same prepared weights
    xs = (data ^ 0x80).view(np.int8)
    bias = rng.uniform_s8((K,), 5).astype(np.int32) * 313
    if N != 32:
        ref_f = oracle.conv2d_nchwc_int8_fused(xs, wt, bias, 5, stride, pad, dil, conv=oracle.c_conv2d_nchwc)
        out = U.conv2d_NCHWc_int8_fused(_t(xs, dev), p, _t(bias, dev), 5, stride, pad, dil, "int32", "NCHW4c", "NCHW16c")
        torch.cuda.synchronize()
        assert U.last_variant().startswith("s8prep_c4")
        assert np.array_equal(out.cpu().numpy(), ref_f), U.last_variant()


def test_conv2d_prepared_c4_every_direct_variant(dev, oracle, monkeypatch):
    from unit_amd import _lib
    N, C, H, W, K = 2, 8, 13, 17, 96
    data = rng.uniform_u8((N, C // 4, H, W, 4), 21)
    wt = rng.uniform_s8((K // 16, C // 4, 7, 7, 1, 16, 4), 22)
    ref = oracle.c_conv2d_nchwc(data, wt, 2, 3, 1)
    d = _t(data, dev)
    p = U.prepare_conv2d_weight(_t(wt, dev))
    names = set()
    for v in range(1, _lib.load().unit_conv_variant_count() + 1):
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        out = U.conv2d_NCHWc_int8(d, p, 2, 3, 1, "int32", "NCHW4c")
        torch.cuda.synchronize()
        names.add(U.last_variant())
        assert np.array_equal(out.cpu().numpy(), ref), (v, U.last_variant())
    assert len(names) >= 15 and all(n.startswith("i8prep_c4") for n in names), names


@pytest.mark.parametrize("N,C,H,W,K,ks,stride,pad", [
    (2, 80, 9, 11, 96, 3, 1, 1),    # 45 taps: odd, zero padding, ragged tiles
    (1, 32, 5, 5, 16, 1, 1, 0),     # one k-step: k-groups beyond the first have nothing to do
    (3, 256, 7, 7, 160, 3, 2, 1),   # a long reduction over few pixels
    (1, 48, 8, 8, 32, 3, 1, 0),     # 27 taps without padding
    (2, 16, 12, 12, 32, 3, 1, (2, 2, 2)),          # dilation 2 (third entry of the padding triple), padding 2
    (1, 48, 10, 10, 80, 5, (2, 1), ((2, 0), 1)),   # 5 x 5 window (25 positions), anisotropic stride and padding
])
def test_conv2d_prepared_every_direct_variant(dev, oracle, monkeypatch, N, C, H, W, K, ks, stride, pad):
    """u8 and fused signed form on every direct and every LDS-shared variant (ids of register-staged variants fall
    back to a direct one)."""
    from unit_amd import _lib
    dil = 1
    if isinstance(pad, tuple) and len(pad) == 3:    # (pad, pad, dilation)
        pad, dil = pad[0], pad[2]
    elif isinstance(pad, tuple) and isinstance(pad[0], tuple):  # ((pad_h, pad_w), dilation)
        pad, dil = pad
    data = rng.uniform_u8((N, C // 16, H, W, 16), 11 * C + H)
    xs = (data ^ 0x80).view(np.int8)
    wt = rng.uniform_s8((K // 16, C // 16, ks, ks, 4, 16, 4), 5 * K + ks)
    bias = rng.uniform_s8((K,), 5).astype(np.int32) * 1001
    ref = oracle.c_conv2d_nchwc(data, wt, stride, pad, dil)
    ref_fused = oracle.conv2d_nchwc_int8_fused(xs, wt, bias, -7, stride, pad, dil, conv=oracle.c_conv2d_nchwc)
    d, x, tb = _t(data, dev), _t(xs, dev), _t(bias, dev)
    p = U.prepare_conv2d_weight(_t(wt, dev))
    names = set()
    for v in range(1, _lib.load().unit_conv_variant_count() + 1):
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        out = U.conv2d_NCHWc_int8(d, p, stride, pad, dil)
        torch.cuda.synchronize()
        names.add(U.last_variant())
        assert np.array_equal(out.cpu().numpy(), ref), (v, U.last_variant())
        out = U.conv2d_NCHWc_int8_fused(x, p, tb, -7, stride, pad, dil)
        torch.cuda.synchronize()
        names.add(U.last_variant())
        assert np.array_equal(out.cpu().numpy(), ref_fused), (v, U.last_variant())
    assert len(names) >= 30 and all(n.startswith(("i8prep", "s8prep", "i8lds", "s8lds")) for n in names), names
    assert sum(n.startswith("i8lds") for n in names) >= 4 and sum(n.startswith("s8lds") for n in names) >= 4, names


FP16_CASES = [
    # N, C, H, W, K, kernel, stride
    (1, 64, 16, 18, 64, 3, 1),
    (1, 16, 9, 9, 16, 1, 1),
    (2, 32, 12, 10, 48, 3, 2),
    (1, 256, 30, 30, 256, 3, 2),
    (4, 128, 30, 30, 128, 3, 1),
    (32, 256, 16, 16, 256, 3, 1),
]


@pytest.mark.parametrize("N,C,H,W,K,ks,stride", FP16_CASES)
def test_conv2d_fp16_prepared(dev, oracle, N, C, H, W, K, ks, stride):
    a = rng.normal_f16((N, C // 16, H, W, 16), 5 + C)
    b = rng.normal_f16((K // 16, C // 16, ks, ks, 16, 16), 9 + K, 1.0 / np.sqrt(C * ks * ks))
    ta = _t(a, dev)
    out = U.conv2d_NCHW16c_OHWI16o(ta, U.prepare_conv2d_weight(_t(b, dev)), stride, stride, "float32")
    torch.cuda.synchronize()
    assert U.last_variant().startswith("f16prep")
    ref = oracle.conv2d_nchw16c_f16(a, b, stride, stride)
    assert tuple(out.shape) == ref.shape
    floor = 1e-3 * np.abs(ref).max()
    err = float((np.abs(out.cpu().numpy().astype(np.float64) - ref) / np.maximum(np.abs(ref), floor)).max())
    assert err <= REL_TOL, (err, U.last_variant())


@pytest.mark.parametrize("N,C,H,W,K,ks,stride", [(2, 80, 9, 11, 96, 3, 1),    # 45 taps: a surplus k-step in the last stage
                                                 (1, 32, 12, 10, 48, 3, 2),   # stride 2
                                                 (3, 64, 7, 7, 160, 1, 1)])   # 1 x 1: four k-steps, three images
def test_conv2d_fp16_prepared_every_direct_variant(dev, oracle, monkeypatch, N, C, H, W, K, ks, stride):
    """Integer-valued data: fp32 accumulation is exact in any order, so every variant -- direct and LDS-shared -- must
    reproduce the float64 reference bit for bit; and on random data the prepared and the plain convolution of one
    direct variant agree bit for bit (same products, same summation order)."""
    from unit_amd import _lib
    a = (rng.uniform_u8((N, C // 16, H, W, 16), 3 + C) % 7).astype(np.float16) - 3
    b = (rng.uniform_u8((K // 16, C // 16, ks, ks, 16, 16), 4 + K) % 5).astype(np.float16) - 2
    ra = rng.normal_f16(a.shape, 1)
    rb = rng.normal_f16(b.shape, 2, 0.05)
    ref = oracle.conv2d_nchw16c_f16(a, b, stride, stride)
    ta, tra, trb = _t(a, dev), _t(ra, dev), _t(rb, dev)
    p, rp = U.prepare_conv2d_weight(_t(b, dev)), U.prepare_conv2d_weight(trb)
    names = set()
    for v in range(1, _lib.load().unit_conv_variant_count() + 1):
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        try:
            out = U.conv2d_NCHW16c_OHWI16o(ta, p, stride, stride)
        except ValueError as e:  # a variant may only be refused for its LDS budget (parked fp32 partial tiles)
            assert "LDS" in str(e), (v, str(e))
            continue
        torch.cuda.synchronize()
        names.add(U.last_variant())
        assert np.array_equal(out.cpu().numpy().astype(np.float64), ref), (v, U.last_variant())
        plain = U.conv2d_NCHW16c_OHWI16o(tra, trb, stride, stride)
        if U.last_variant().startswith("f16direct"):
            prep = U.conv2d_NCHW16c_OHWI16o(tra, rp, stride, stride)
            torch.cuda.synchronize()
            if U.last_variant().startswith("f16prep"):  # the same direct variant on both layouts
                assert torch.equal(plain, prep), (v, U.last_variant())
            else:                                        # an LDS-shared variant sums in another order
                assert float((plain - prep).abs().max()) <= 1e-2 * float(plain.abs().max()), (v, U.last_variant())
    assert len(names) >= 15 and all(n.startswith(("f16prep", "f16lds")) for n in names), names
    assert sum(n.startswith("f16lds") for n in names) >= 4, names


def test_misaligned_views_are_rejected(dev):
    """A tensor view that starts 8 bytes into an allocation: the library refuses it instead of issuing
    misaligned 16-byte accesses."""
    flat = _t(rng.uniform_u8((1 * 2 * 8 * 8 * 16 + 8,), 3), dev)
    data = flat[8:].view(1, 2, 8, 8, 16)
    assert data.data_ptr() % 16 == 8
    wt = _t(rng.uniform_s8((2, 2, 3, 3, 4, 16, 4), 1), dev)
    with pytest.raises(ValueError, match="aligned"):
        U.conv2d_NCHWc_int8(data, wt, 1, 1)
    with pytest.raises(ValueError, match="aligned"):
        U.conv2d_NCHWc_int8(data, U.prepare_conv2d_weight(wt), 1, 1)


def test_prepared_rejections(dev):
    wt = _t(rng.uniform_s8((2, 2, 3, 3, 4, 16, 4), 1), dev)
    p = U.prepare_conv2d_weight(wt)
    with pytest.raises(ValueError):   # channel count of the data does not match
        U.conv2d_NCHWc_int8(_t(rng.uniform_u8((1, 3, 8, 8, 16), 2), dev), p, 1, 1)
    with pytest.raises(TypeError):    # int8 weights into the fp16 operator
        U.conv2d_NCHW16c_OHWI16o(_t(rng.normal_f16((1, 2, 8, 8, 16), 3), dev), p, 1, 1)
    with pytest.raises(ValueError):   # 4-channel blocks: KW <= 8 only
        U.prepare_conv2d_weight(_t(rng.uniform_s8((2, 1, 3, 9, 1, 16, 4), 1), dev))
    with pytest.raises(ValueError):   # prepared for 4-channel blocks, data in 16-channel blocks
        p4 = U.prepare_conv2d_weight(_t(rng.uniform_s8((2, 4, 3, 3, 1, 16, 4), 1), dev))
        U.conv2d_NCHWc_int8(_t(rng.uniform_u8((1, 1, 8, 8, 16), 2), dev), p4, 1, 1)


REQUANT_CASES = [
    # N, C, H, W, K, kernel, stride, pad, scale, shift, with bias
    (1, 64, 56, 56, 64, 3, 1, 1, 3, 12, True),
    (2, 32, 9, 7, 48, 3, 1, 1, 1, 9, False),          # K not a multiple of 32: the last plane pair is half empty
    (3, 64, 14, 14, 128, 1, 1, 0, -5, 11, True),      # negative scale
    (1, 512, 7, 7, 512, 3, 1, 1, 77, 20, True),       # k-groups: partial tiles summed in LDS first
    (2, 80, 9, 11, 96, 3, 2, (1, 0, 2, 1), 1 << 30, 45, True),   # 64-bit product and shift
    (1, 4, 32, 32, 64, 7, 2, 3, 9, 12, True),         # 4-channel stem
    (32, 64, 56, 56, 256, 1, 1, 0, 5, 13, True),      # ResNet-50 batch 32, output-bound layer
    (1, 16, 8, 8, 16, 1, 1, 0, 1, 1, False),          # shift 1
]


def test_conv2d_fp16_prepared_large_window_keeps_direct_kernels(dev, oracle, monkeypatch):
    """A 7 x 7 window has 49 positions, more than the 32-bit position set of the LDS-shared kernels holds: whatever
    variant is forced, the prepared fp16 convolution runs a direct kernel, and integer-valued data reproduces the
    float64 reference bit for bit."""
    from unit_amd import _lib
    N, C, H, W, K, ks = 1, 16, 12, 13, 32, 7
    a = (rng.uniform_u8((N, C // 16, H, W, 16), 61) % 7).astype(np.float16) - 3
    b = (rng.uniform_u8((K // 16, C // 16, ks, ks, 16, 16), 62) % 5).astype(np.float16) - 2
    ref = oracle.conv2d_nchw16c_f16(a, b, 1, 1)
    ta, p = _t(a, dev), U.prepare_conv2d_weight(_t(b, dev))
    L = _lib.load()
    for v in range(1, L.unit_conv_variant_count() + 1):
        if L.unit_conv_variant_is_direct(v - 1) != 2:
            continue
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        out = U.conv2d_NCHW16c_OHWI16o(ta, p, 1, 1)
        torch.cuda.synchronize()
        assert U.last_variant().startswith("f16prep"), (v, U.last_variant())
        assert np.array_equal(out.cpu().numpy().astype(np.float64), ref), (v, U.last_variant())


@pytest.mark.parametrize("N,C,H,W,K,ks,stride,pad,scale,shift,with_bias", REQUANT_CASES)
def test_conv2d_requant_u8(dev, oracle, N, C, H, W, K, ks, stride, pad, scale, shift, with_bias):
    """Requantised u8 output against the oracle's integer definition (bit-exact), on inputs scaled so that the
    results spread over the whole 0..255 range and both clamps."""
    cb = 16 if C % 16 == 0 else 4
    data = rng.uniform_u8((N, C // cb, H, W, cb), 7 * C + H)
    wt = rng.uniform_s8((K // 16, C // cb, ks, ks, cb // 4, 16, 4), 3 * K + ks)
    bias = rng.uniform_s8((K,), 5).astype(np.int32) * 20011 if with_bias else None
    ref = oracle.conv2d_nchwc_u8_requant(data, wt, bias, scale, shift, stride, pad, 1, conv=oracle.c_conv2d_nchwc)
    out = U.conv2d_NCHWc_int8_requant(_t(data, dev), U.prepare_conv2d_weight(_t(wt, dev)),
                                      _t(bias, dev) if with_bias else None, scale, shift, stride, pad)
    torch.cuda.synchronize()
    assert U.last_variant().startswith("q8prep")
    assert out.dtype == torch.uint8 and tuple(out.shape) == ref.shape
    got = out.cpu().numpy()
    assert np.array_equal(got, ref), U.last_variant()


def test_conv2d_requant_every_direct_variant(dev, oracle, monkeypatch):
    from unit_amd import _lib
    N, C, H, W, K, ks = 2, 80, 9, 11, 96, 3
    data = rng.uniform_u8((N, C // 16, H, W, 16), 41)
    wt = rng.uniform_s8((K // 16, C // 16, ks, ks, 4, 16, 4), 42)
    bias = rng.uniform_s8((K,), 43).astype(np.int32) * 3001
    ref = oracle.conv2d_nchwc_u8_requant(data, wt, bias, 7, 13, 1, 1, 1, conv=oracle.c_conv2d_nchwc)
    assert 0 < (ref == 0).mean() < 0.9 and (ref == 255).any()   # both clamps and the range in between occur
    d, tb = _t(data, dev), _t(bias, dev)
    p = U.prepare_conv2d_weight(_t(wt, dev))
    names = set()
    for v in range(1, _lib.load().unit_conv_variant_count() + 1):
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        out = U.conv2d_NCHWc_int8_requant(d, p, tb, 7, 13, 1, 1)
        torch.cuda.synchronize()
        names.add(U.last_variant())
        assert np.array_equal(out.cpu().numpy(), ref), (v, U.last_variant())
    assert len(names) >= 15 and sum(n.startswith("q8lds") for n in names) >= 4, names


def test_conv_chain_through_requantised_activations(dev, oracle):
    """Two layers back to back: the u8 output of the first is the input of the second, no layout change."""
    x = rng.uniform_u8((2, 4, 12, 12, 16), 51)
    w1 = rng.uniform_s8((8, 4, 3, 3, 4, 16, 4), 52)
    w2 = rng.uniform_s8((4, 8, 1, 1, 4, 16, 4), 53)
    mid_ref = oracle.conv2d_nchwc_u8_requant(x, w1, None, 3, 14, 1, 1, 1, conv=oracle.c_conv2d_nchwc)
    ref = oracle.c_conv2d_nchwc(mid_ref, w2, 1, 0, 1)
    mid = U.conv2d_NCHWc_int8_requant(_t(x, dev), _t(w1, dev), None, 3, 14, 1, 1)
    out = U.conv2d_NCHWc_int8(mid, U.prepare_conv2d_weight(_t(w2, dev)), 1, 0)
    torch.cuda.synchronize()
    assert np.array_equal(mid.cpu().numpy(), mid_ref) and np.array_equal(out.cpu().numpy(), ref)


def _random_conv_cases(count, seed):
    r = np.random.RandomState(seed)
    cases = []
    while len(cases) < count:
        cb = int(r.choice([4, 16]))
        cc = int(r.randint(1, 4 if cb == 16 else 3))
        kh, kw = int(r.randint(1, 6)), int(r.randint(1, 6))
        sh, sw = int(r.randint(1, 4)), int(r.randint(1, 4))
        pad = tuple(int(x) for x in r.randint(0, 3, size=4))
        h, w = int(r.randint(kh, kh + 14)), int(r.randint(kw, kw + 14))
        dh = int(r.randint(1, 3))
        if (kh - 1) * dh + 1 > h + pad[0] + pad[2]:
            continue
        cases.append((int(r.randint(1, 4)), cc * cb, h, w, 16 * int(r.randint(1, 8)), (kh, kw), (sh, sw), pad, (dh, 1)))
    return cases


@pytest.mark.parametrize("case", _random_conv_cases(40, 20240521), ids=lambda c: "x".join(str(v) for v in c[:5]))
def test_conv2d_random_shapes_all_forms(dev, oracle, case):
    """Seeded random small configurations (ragged everything: pads, strides, windows, channel counts) through the
    plain, prepared, fused and requantised entry points."""
    N, C, H, W, K, (kh, kw), stride, pad, dil = case
    cb = 16 if C % 16 == 0 else 4
    seed = N + 3 * C + 5 * H + 7 * W + 11 * K + 13 * kh + 17 * kw
    data = rng.uniform_u8((N, C // cb, H, W, cb), seed)
    wt = rng.uniform_s8((K // 16, C // cb, kh, kw, cb // 4, 16, 4), seed + 1)
    bias = rng.uniform_s8((K,), seed + 2).astype(np.int32) * 997
    ref = oracle.c_conv2d_nchwc(data, wt, stride, pad, dil)
    d, w, tb = _t(data, dev), _t(wt, dev), _t(bias, dev)
    layout = f"NCHW{cb}c"
    out = U.conv2d_NCHWc_int8(d, w, stride, pad, dil, "int32", layout)
    assert np.array_equal(out.cpu().numpy(), ref), ("plain", U.last_variant())
    p = U.prepare_conv2d_weight(w)
    out = U.conv2d_NCHWc_int8(d, p, stride, pad, dil, "int32", layout)
    assert np.array_equal(out.cpu().numpy(), ref), ("prepared", U.last_variant())
    xs = (data ^ 0x80).view(np.int8)
    ref_f = oracle.conv2d_nchwc_int8_fused(xs, wt, bias, 3, stride, pad, dil, conv=oracle.c_conv2d_nchwc)
    for kern in (w, p):
        out = U.conv2d_NCHWc_int8_fused(_t(xs, dev), kern, tb, 3, stride, pad, dil, "int32", layout)
        assert np.array_equal(out.cpu().numpy(), ref_f), ("fused", U.last_variant())
    ref_q = oracle.conv2d_nchwc_u8_requant(data, wt, bias, 5, 11, stride, pad, dil, conv=oracle.c_conv2d_nchwc)
    out = U.conv2d_NCHWc_int8_requant(d, p, tb, 5, 11, stride, pad, dil)
    assert np.array_equal(out.cpu().numpy(), ref_q), ("requant", U.last_variant())


def _random_fp16_cases(count, seed):
    r = np.random.RandomState(seed)
    return [(int(r.randint(1, 4)), 16 * int(r.randint(1, 5)), int(r.randint(5, 20)), int(r.randint(5, 20)),
             16 * int(r.randint(1, 7)), int(r.randint(1, 5)), int(r.randint(1, 3))) for _ in range(count)]


@pytest.mark.parametrize("N,C,H,W,K,ks,stride", _random_fp16_cases(16, 77))
def test_conv2d_fp16_random_shapes(dev, oracle, N, C, H, W, K, ks, stride):
    a = rng.normal_f16((N, C // 16, H, W, 16), N + C + H)
    b = rng.normal_f16((K // 16, C // 16, ks, ks, 16, 16), K + ks, 1.0 / np.sqrt(C * ks * ks))
    ta, tb = _t(a, dev), _t(b, dev)
    plain = U.conv2d_NCHW16c_OHWI16o(ta, tb, stride, stride)
    prep = U.conv2d_NCHW16c_OHWI16o(ta, U.prepare_conv2d_weight(tb), stride, stride)
    torch.cuda.synchronize()
    ref = oracle.conv2d_nchw16c_f16(a, b, stride, stride)
    floor = 1e-3 * np.abs(ref).max()
    for out in (plain, prep):
        err = float((np.abs(out.cpu().numpy().astype(np.float64) - ref) / np.maximum(np.abs(ref), floor)).max())
        assert err <= REL_TOL, (err, U.last_variant())
