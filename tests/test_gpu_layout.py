"""Layout transforms and weight pre-packs on the GPU: byte-exact against the oracle."""
import numpy as np
import pytest
import torch

import unit_amd as U
from unit_amd import rng

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.parametrize("shape,cb", [((2, 64, 14, 14), 16), ((1, 3, 224, 224), 4), ((1, 35, 7, 9), 16),
                                      ((3, 10, 5, 5), 4), ((32, 256, 56, 56), 16),
                                      ((2, 40, 8, 8), 16),     # 16-pixel groups, channel tail in the last block
                                      ((1, 16, 4, 4), 16),     # one 16-pixel group
                                      ((3, 100, 12, 20), 16),
                                      ((32, 512, 7, 7), 16),    # 49-pixel planes: three full groups and one pixel
                                      ((5, 33, 7, 7), 16),      # ... with a channel tail
                                      ((2, 64, 17, 17), 16),    # odd plane size, unaligned plane starts
                                      ((3, 20, 3, 5), 16),      # planes smaller than a group
                                      ((1, 16, 1, 1), 16),
                                      ((1, 2000, 5, 6), 16),    # many planes, groups of 16 + 14
                                      ((32, 128, 28, 28), 16)])
def test_pack_unpack_u8(dev, oracle, shape, cb):
    x = rng.uniform_u8(shape, 1)
    p = U.pack_nchwc(_t(x, dev), cb)
    assert np.array_equal(p.cpu().numpy(), oracle.pack_nchwc(x, cb))
    back = U.unpack_nchwc(p, shape[1])
    assert np.array_equal(back.cpu().numpy(), x)


@pytest.mark.parametrize("dtype", [np.float16, np.int32])
@pytest.mark.parametrize("shape", [(2, 32, 6, 6), (1, 48, 7, 7), (4, 64, 28, 28)])
def test_pack_unpack_wide(dev, oracle, dtype, shape):
    x = rng.random_bytes(int(np.prod(shape)) * np.dtype(dtype).itemsize, 3).view(dtype).reshape(shape)
    if dtype == np.float16:
        x = np.nan_to_num(x, nan=1.0)
    p = U.pack_nchwc(_t(x, dev), 16)
    assert np.array_equal(p.cpu().numpy().view(np.uint8), oracle.pack_nchwc(x, 16).view(np.uint8))
    assert np.array_equal(U.unpack_nchwc(p).cpu().numpy().view(np.uint8), x.view(np.uint8))


@pytest.mark.parametrize("o,i,ks,cb", [(64, 64, 3, 16), (64, 3, 7, 4), (40, 35, 3, 16), (2048, 1024, 1, 16)])
def test_prepack_conv_weight(dev, oracle, o, i, ks, cb):
    w = rng.uniform_s8((o, i, ks, ks), 9)
    out = U.prepack_conv_weight(_t(w, dev), cb).cpu().numpy()
    assert np.array_equal(out, oracle.prepack_conv_weight(w, cb))


def test_prepack_dense_and_f16(dev, oracle):
    w = rng.uniform_s8((384, 272), 4)
    assert np.array_equal(U.prepack_dense_weight(_t(w, dev)).cpu().numpy(), oracle.prepack_dense_weight(w))
    wf = rng.normal_f16((32, 48, 3, 3), 8)
    assert np.array_equal(U.prepack_conv_weight_f16(_t(wf, dev)).cpu().numpy(), oracle.prepack_conv_weight_f16(wf))


def test_nchw_end_to_end(dev, oracle):
    """NCHW u8 -> pack -> conv -> unpack equals the textbook NCHW / OIHW convolution."""
    N, C, H, K = 2, 35, 12, 40
    x = rng.uniform_u8((N, C, H, H), 21)
    w = rng.uniform_s8((K, C, 3, 3), 22)
    out5 = U.conv2d_NCHWc_int8(U.pack_nchwc(_t(x, dev), 16), U.prepack_conv_weight(_t(w, dev), 16), 1, 1)
    out = U.unpack_nchwc(out5, K).cpu().numpy()
    ref = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), padding=1)
    assert np.array_equal(out.astype(np.float64), ref.numpy())
