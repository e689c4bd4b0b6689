"""The Relay-level graph (conv2d + bias) * multiplier, NCHW int8 in and NCHW int32 out
(apps/cpu/relay/conv2d.py:15-27, legalised form apps/cpu/relay/result.log:3-26 and :6803-6828), through
the C ABI: bit-exact against a plain NCHW integer convolution (float64 on the CPU, exact at these
magnitudes -- a check that does not go through any blocked layout) and against the oracle's operators
composed the way the graph composes them."""
import os

import numpy as np
import pytest
import torch

import unit_amd as U
from oracle import oracle as O
from unit_amd import relay, rng

pytestmark = pytest.mark.gpu


def _i32(shape, seed, lo, hi):
    return np.random.default_rng(seed).integers(lo, hi, shape, dtype=np.int32)


def _plain_graph(x, w, b, mult, stride, padding, dilation=1):
    y = torch.nn.functional.conv2d(torch.from_numpy(x.astype(np.float64)), torch.from_numpy(w.astype(np.float64)),
                                   stride=stride, padding=padding, dilation=dilation).numpy()
    y = np.rint(y).astype(np.int64)
    if b is not None:
        y = y + b.reshape(1, -1, 1, 1).astype(np.int64)
    y = y * mult
    assert np.abs(y).max() < 2 ** 31
    return y.astype(np.int32)


CASES = [
    # n, ic, h, w, oc, kh, kw, stride, padding
    (1, 64, 14, 14, 64, 3, 3, 1, 0),
    (2, 3, 37, 41, 64, 7, 7, 2, 0),      # the stem's form: 3 -> 4 channels, NCHW4c
    (2, 3, 32, 32, 64, 7, 7, 2, 3),
    (3, 32, 9, 11, 40, 3, 3, 1, 1),      # output channels padded 40 -> 48, not written back
    (1, 8, 12, 12, 16, 3, 3, 1, 1),      # two 4-channel blocks
    (2, 20, 10, 10, 24, 1, 1, 2, 0),     # five 4-channel blocks
    (1, 128, 7, 7, 200, 1, 1, 1, 0),     # 49 pixels per image: planes not a multiple of 4 pixels
    (5, 16, 7, 7, 32, 3, 3, 1, 1),       # 32-pixel blocks straddle images
    (1, 1024, 16, 16, 2048, 1, 1, 1, 0),  # the graph printed at result.log:3-26
]


@pytest.mark.parametrize("n,ic,h,w,oc,kh,kw,stride,padding", CASES)
def test_graph_bit_exact(dev, n, ic, h, w, oc, kh, kw, stride, padding):
    x = rng.uniform_s8((n, ic, h, w), 11 + ic)
    wt = rng.uniform_s8((oc, ic, kh, kw), 12 + oc)
    b = _i32((1, oc, 1, 1), 13, -5000, 5000)
    want = _plain_graph(x, wt, b, 11, stride, padding)
    g = relay.Conv2dBiasMultiply(torch.from_numpy(wt).to(dev), torch.from_numpy(b).to(dev), 11, stride, padding)
    xd = torch.from_numpy(x).to(dev)
    got = g(xd)
    assert "_nchw" in U.last_variant()
    assert got.shape == want.shape and got.dtype == torch.int32
    assert np.array_equal(got.cpu().numpy(), want)
    unfolded = g(xd, fold_output_transform=False)
    assert torch.equal(unfolded, got)


def test_graph_matches_oracle_composition(dev):
    """Ops #0-#6 of result.log:30-36 composed from the oracle's operators."""
    n, ic, h, w, oc, ks = 2, 32, 10, 10, 48, 3
    x = rng.uniform_s8((n, ic, h, w), 1)
    wt = rng.uniform_s8((oc, ic, ks, ks), 2)
    b = _i32((oc,), 3, -999, 999)
    data = O.pack_nchwc(x, 16)
    wp = O.prepack_conv_weight(wt, 16)
    out = O.conv2d_nchwc_int8_fused(data, wp, b, 11, 1, 0, 1)
    want = O.unpack_nchwc(out, oc)
    g = relay.Conv2dBiasMultiply(torch.from_numpy(wt).to(dev), torch.from_numpy(b).to(dev), 11, 1, 0)
    assert np.array_equal(g(torch.from_numpy(x).to(dev)).cpu().numpy(), want)
    assert np.array_equal(want, _plain_graph(x, wt, b, 11, 1, 0))


def test_graph_without_bias_and_negative_multiplier(dev):
    x = rng.uniform_s8((1, 16, 8, 8), 5)
    wt = rng.uniform_s8((16, 16, 3, 3), 6)
    g = relay.Conv2dBiasMultiply(torch.from_numpy(wt).to(dev), None, -3, 1, 1)
    assert np.array_equal(g(torch.from_numpy(x).to(dev)).cpu().numpy(), _plain_graph(x, wt, None, -3, 1, 1))


def test_planar_store_on_every_direct_variant(dev):
    """Every direct kernel variant writes the same NCHW result (one wave per tile, k-groups summed in LDS)."""
    from unit_amd import _lib
    L = _lib.load()
    n, ic, h, w, oc = 3, 64, 9, 9, 72
    x = rng.uniform_s8((n, ic, h, w), 21)
    wt = rng.uniform_s8((oc, ic, 3, 3), 22)
    b = _i32((oc,), 23, -999, 999)
    want = _plain_graph(x, wt, b, 7, 1, 1)
    g = relay.Conv2dBiasMultiply(torch.from_numpy(wt).to(dev), torch.from_numpy(b).to(dev), 7, 1, 1)
    xd = torch.from_numpy(x).to(dev)
    saved = os.environ.get("UNIT_AMD_CONV_VARIANT")
    ran = 0
    try:
        for v in range(L.unit_conv_variant_count()):
            if L.unit_conv_variant_is_direct(v) not in (1, 2):  # direct and LDS-shared variants take prepared weights
                continue
            os.environ["UNIT_AMD_CONV_VARIANT"] = str(v + 1)
            try:
                got = g(xd)
            except ValueError as e:  # the variant's LDS need exceeds the budget
                assert "LDS" in str(e)
                continue
            assert np.array_equal(got.cpu().numpy(), want), U.last_variant()
            ran += 1
    finally:
        if saved is None:
            os.environ.pop("UNIT_AMD_CONV_VARIANT", None)
        else:
            os.environ["UNIT_AMD_CONV_VARIANT"] = saved
    assert ran >= 8


def test_planar_needs_prepared_weights_and_a_matching_channel_count(dev):
    data = torch.zeros((1, 1, 4, 4, 16), dtype=torch.int8, device=dev)
    wt = torch.zeros((2, 1, 1, 1, 4, 16, 4), dtype=torch.int8, device=dev)
    with pytest.raises(ValueError, match="prepared"):
        U.conv2d_NCHWc_int8_fused(data, wt, None, 1, 1, 0, out_layout="NCHW")
    p = U.prepare_conv2d_weight(wt)
    for bad in (16, 33, 0):
        with pytest.raises(ValueError, match="out_channels"):
            U.conv2d_NCHWc_int8_fused(data, p, None, 1, 1, 0, out_layout="NCHW", out_channels=bad)
    assert U.conv2d_NCHWc_int8_fused(data, p, None, 1, 1, 0, out_layout="NCHW", out_channels=17).shape == (1, 17, 4, 4)


def test_driver_prints_a_time(dev, capsys):
    assert relay.main("1 32 14 14 32 32 3 3 1 1".split()) == 0
    out = capsys.readouterr().out
    assert " us per run" in out


def test_graph_replay_follows_the_input(dev):
    wt = rng.uniform_s8((32, 16, 3, 3), 31)
    g = relay.Conv2dBiasMultiply(torch.from_numpy(wt).to(dev), None, 5, 1, 1)
    x1, x2 = rng.uniform_s8((2, 16, 9, 9), 32), rng.uniform_s8((2, 16, 9, 9), 33)
    xd = torch.from_numpy(x1).to(dev)
    replay = g.graph(xd)
    for x in (x1, x2, x1):  # eager work and synchronisations between the replays
        xd.copy_(torch.from_numpy(x).to(dev))
        torch.cuda.synchronize()
        assert np.array_equal(replay().cpu().numpy(), _plain_graph(x, wt, None, 5, 1, 1))
