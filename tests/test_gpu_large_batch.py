"""Activations beyond 2^31-1 bytes: the kernels address with 32-bit offsets, so the C ABI runs such a convolution (or
layout transform) as several launches over slices of the batch.  Each case checks, against the oracle, the images on
both sides of every slice boundary plus the first and the last ones; inputs are drawn on the GPU (seeded) and only
the checked images cross to the host."""
import numpy as np
import pytest
import torch

import unit_amd as U
from unit_amd import rng

pytestmark = pytest.mark.gpu

LIMIT = 2 ** 31 - 1
REL_TOL = 1e-2


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _windows(n, image_bytes):
    """Image ranges to check: around every slice boundary (a slice holds LIMIT // image_bytes images), head, tail."""
    per = LIMIT // image_bytes
    assert per < n, "the case does not exceed the limit"
    spans = [(0, 2), (n - 2, n)]
    spans += [(b - 2, min(b + 2, n)) for b in range(per, n, per)]
    return spans


def _randint_u8(shape, seed, dev):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    return torch.randint(0, 256, shape, dtype=torch.uint8, device=dev, generator=g)


def test_int32_output_beyond_the_limit(dev, oracle):
    """1x1 64 -> 256 on 56 x 56, 700 images: 2.25 GB of int32 results.  Reference weight layout, prepared weights, the
    fused signed form and its NCHW store (250 of 256 channels)."""
    n, c, k, hw = 700, 64, 256, 56
    data = _randint_u8((n, c // 16, hw, hw, 16), 4101, dev)
    wt = rng.uniform_s8((k // 16, c // 16, 1, 1, 4, 16, 4), 4102)
    bias = rng.uniform_s8((k,), 4103).astype(np.int32) * 1000
    tw, tb = _t(wt, dev), _t(bias, dev)
    wp = U.prepare_conv2d_weight(tw)
    spans = _windows(n, hw * hw * k * 4)
    for kernel in (tw, wp):
        out = U.conv2d_NCHWc_int8(data, kernel, 1, 0)
        assert out.numel() * 4 > LIMIT
        for a, b in spans:
            ref = oracle.c_conv2d_nchwc(data[a:b].cpu().numpy(), wt, 1, 0, 1)
            assert np.array_equal(out[a:b].cpu().numpy(), ref), (a, b, U.last_variant())
        del out
    data_s8 = data.view(torch.int8)
    fused = U.conv2d_NCHWc_int8_fused(data_s8, wp, tb, 11, 1, 0)
    for a, b in spans:
        ref = oracle.conv2d_nchwc_int8_fused(data_s8[a:b].cpu().numpy(), wt, bias, 11, 1, 0, 1, conv=oracle.c_conv2d_nchwc)
        assert np.array_equal(fused[a:b].cpu().numpy(), ref), (a, b, U.last_variant())
    del fused
    planar = U.conv2d_NCHWc_int8_fused(data_s8, wp, tb, 11, 1, 0, out_layout="NCHW", out_channels=250)
    assert tuple(planar.shape) == (n, 250, hw, hw)
    for a, b in spans:  # sliced where the blocked result would be
        ref = oracle.conv2d_nchwc_int8_fused(data_s8[a:b].cpu().numpy(), wt, bias, 11, 1, 0, 1, conv=oracle.c_conv2d_nchwc)
        assert np.array_equal(planar[a:b].cpu().numpy(), oracle.unpack_nchwc(ref, 250)), (a, b, U.last_variant())


def test_u8_input_beyond_the_limit_requantised(dev, oracle):
    """1x1 stride 2, 256 -> 16 on 56 x 56, 2700 images: 2.17 GB of u8 data, small u8 result."""
    n, c, k, hw = 2700, 256, 16, 56
    data = _randint_u8((n, c // 16, hw, hw, 16), 4201, dev)
    assert data.numel() > LIMIT
    wt = rng.uniform_s8((k // 16, c // 16, 1, 1, 4, 16, 4), 4202)
    bias = rng.uniform_s8((k,), 4203).astype(np.int32) * 1000
    wp = U.prepare_conv2d_weight(_t(wt, dev))
    q = U.conv2d_NCHWc_int8_requant(data, wp, _t(bias, dev), 3, 16, 2, 0)
    for a, b in _windows(n, c * hw * hw):
        ref = oracle.conv2d_nchwc_u8_requant(data[a:b].cpu().numpy(), wt, bias, 3, 16, 2, 0, 1, conv=oracle.c_conv2d_nchwc)
        assert np.array_equal(q[a:b].cpu().numpy(), ref), (a, b, U.last_variant())


def test_fp16_input_beyond_the_limit(dev, oracle):
    """fp16 1x1 stride 2, 256 -> 16 on 56 x 56, 1400 images (2.25 GB of data), both weight layouts."""
    n, c, k, hw = 1400, 256, 16, 56
    g = torch.Generator(device=dev)
    g.manual_seed(4301)
    a16 = torch.randn((n, c // 16, hw, hw, 16), dtype=torch.float16, device=dev, generator=g)
    assert a16.numel() * 2 > LIMIT
    b16 = rng.normal_f16((k // 16, c // 16, 1, 1, 16, 16), 4302, 1.0 / np.sqrt(c))
    tb = _t(b16, dev)
    for kernel in (tb, U.prepare_conv2d_weight(tb)):
        out = U.conv2d_NCHW16c_OHWI16o(a16, kernel, 2, 2, "float32")
        for a, b in _windows(n, c * hw * hw * 2):
            ref = oracle.conv2d_nchw16c_f16(a16[a:b].cpu().numpy(), b16, 2, 2)
            got = out[a:b].cpu().numpy()
            rel = np.abs(got - ref) / np.maximum(np.abs(ref), 1e-3 * np.abs(ref).max())
            assert float(rel.max()) <= REL_TOL, (a, b, U.last_variant())


def test_layout_kernels_beyond_the_limit(dev, oracle):
    """pack and unpack of 2700 x 250 x 56 x 56 bytes (channels padded to 256: 2.17 GB blocked)."""
    n, c, hw = 2700, 250, 56
    x = _randint_u8((n, c, hw, hw), 4401, dev).view(torch.int8)
    packed = U.pack_nchwc(x, 16)
    assert packed.numel() > LIMIT
    for a, b in _windows(n, 256 * hw * hw):
        assert np.array_equal(packed[a:b].cpu().numpy(), oracle.pack_nchwc(x[a:b].cpu().numpy(), 16)), (a, b)
    back = U.unpack_nchwc(packed, c)
    del packed
    for a, b in _windows(n, 256 * hw * hw):
        assert torch.equal(back[a:b], x[a:b]), (a, b)


def _row_windows(m, row_bytes):
    per = LIMIT // row_bytes // 256 * 256  # slices are whole tiles of 256 rows
    assert per < m, "the case does not exceed the limit"
    return [(0, 4), (m - 4, m)] + [(b - 4, min(b + 4, m)) for b in range(per, m, per)]


def test_gemm_results_beyond_the_limit(dev, oracle):
    """70000 x 8192 results (2.29 GB of int32 / fp32) from a 64-long reduction: the int8 dense on both weight layouts
    and the fp16 GEMM on both layouts of b run as slices of rows."""
    m, n, k = 70000, 8192, 64
    a = _randint_u8((m, k), 4501, dev)
    w = rng.uniform_s8((n, k), 4502)
    spans = _row_windows(m, n * 4)
    for out in (U.dense(a, _t(w, dev)), U.dense_dotprod(a, _t(oracle.prepack_dense_weight(w), dev))):
        assert out.numel() * 4 > LIMIT
        for r0, r1 in spans:
            assert np.array_equal(out[r0:r1].cpu().numpy(), oracle.dense_logical(a[r0:r1].cpu().numpy(), w)), (r0, r1)
        del out
    g = torch.Generator(device=dev)
    g.manual_seed(4503)
    a16 = torch.randn((m, k), dtype=torch.float16, device=dev, generator=g)
    b16 = rng.normal_f16((k, n), 4504, 1.0 / np.sqrt(k))
    tb = _t(b16, dev)
    for b_arg in (tb, U.prepare_gemm_b(tb)):
        out = U.gemm_fp16(a16, b_arg)
        for r0, r1 in spans:
            ref = oracle.gemm_f16(a16[r0:r1].cpu().numpy(), b16)
            rel = np.abs(out[r0:r1].cpu().numpy() - ref) / np.maximum(np.abs(ref), 1e-3 * np.abs(ref).max())
            assert float(rel.max()) <= REL_TOL, (r0, r1, U.last_variant())
        del out


def test_conv3d_results_beyond_the_limit(dev, oracle):
    """conv3d 16 -> 64 channels, 2 x 2 x 2 window on 8 x 56 x 56 volumes, 420 of them: 2.28 GB of int32 results."""
    n, c, k, dd, hw = 420, 16, 64, 8, 56
    data = _randint_u8((n, 1, dd, hw, hw, 16), 4601, dev).view(torch.int8)
    wt = rng.uniform_s8((k // 16, 1, 2, 2, 2, 4, 16, 4), 4602)
    out = U.conv3d_NCDHWc_int8(data, _t(wt, dev), 1)
    assert out.numel() * 4 > LIMIT
    for a, b in _windows(n, 7 * 55 * 55 * k * 4):
        assert np.array_equal(out[a:b].cpu().numpy(), oracle.conv3d_ncdhwc_int8(data[a:b].cpu().numpy(), wt, 1)), (a, b)
