"""The benchmark sweeps at their full sizes, every layer bit-exact against the VNNI oracle: ResNet-18 at batch 1 and
ResNet-50 at batch 32 (BASELINE configs 3 and 4; shapes of cpu-shapes.log:368-420), on the reference's weight layout and
on prepared weights."""
import numpy as np
import pytest
import torch

import unit_amd as U
from unit_amd import rng
from unit_amd import workloads as WL

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _layer(s, batch, seed):
    cb = WL.channel_block(s.C)
    cp = -(-s.C // cb) * cb
    data = rng.uniform_u8((batch, cp // cb, s.H, s.W, cb), seed)
    if cp != s.C:
        data[..., s.C % cb:] = 0  # padded input channels hold zeros
    wt = rng.uniform_s8((s.K // 16, cp // cb, s.KH, s.KW, cb // 4, 16, 4), seed + 1)
    return data, wt


@pytest.mark.parametrize("s", WL.RESNET18, ids=lambda s: s.name)
def test_resnet18_batch1_layer(dev, oracle, s):
    data, wt = _layer(s, 1, 7000 + s.C + s.K)
    ref = oracle.c_conv2d_nchwc(data, wt, s.stride, s.pad, 1)
    td, tw = _t(data, dev), _t(wt, dev)
    assert np.array_equal(U.conv2d_NCHWc_int8(td, tw, s.stride, s.pad).cpu().numpy(), ref), U.last_variant()
    if WL.channel_block(s.C) == 16 or s.KW <= 8:
        out = U.conv2d_NCHWc_int8(td, U.prepare_conv2d_weight(tw), s.stride, s.pad)
        assert np.array_equal(out.cpu().numpy(), ref), U.last_variant()


@pytest.mark.parametrize("s", WL.RESNET50, ids=lambda s: s.name)
def test_resnet50_batch32_layer(dev, oracle, s):
    data, wt = _layer(s, 32, 8000 + s.C + s.K)
    ref = torch.from_numpy(oracle.c_conv2d_nchwc(data, wt, s.stride, s.pad, 1))
    td, tw = _t(data, dev), _t(wt, dev)
    out = U.conv2d_NCHWc_int8(td, U.prepare_conv2d_weight(tw), s.stride, s.pad)
    assert torch.equal(out.cpu(), ref), U.last_variant()
    del out
    out = U.conv2d_NCHWc_int8(td, tw, s.stride, s.pad)
    assert torch.equal(out.cpu(), ref), U.last_variant()


@pytest.mark.parametrize("s", WL.RESNET50, ids=lambda s: s.name)
def test_resnet50_batch32_layer_fused_requantised_and_nchw(dev, oracle, s):
    """The same layers in the fused signed form (bias, scale 11: apps/cpu/relay/result.log:3-26), with the NCHW store,
    and requantised to u8, each against the oracle's operator built on the VNNI convolution."""
    data, wt = _layer(s, 32, 9000 + s.C + s.K)
    data_s8 = data.view(np.int8)
    bias = (rng.uniform_s8((s.K,), 9100 + s.K).astype(np.int32) * 1000)
    ref = oracle.conv2d_nchwc_int8_fused(data_s8, wt, bias, 11, s.stride, s.pad, 1, conv=oracle.c_conv2d_nchwc)
    td, tb = _t(data_s8, dev), _t(bias, dev)
    wp = U.prepare_conv2d_weight(_t(wt, dev))
    out = U.conv2d_NCHWc_int8_fused(td, wp, tb, 11, s.stride, s.pad)
    assert torch.equal(out.cpu(), torch.from_numpy(ref)), U.last_variant()
    del out
    planar = U.conv2d_NCHWc_int8_fused(td, wp, tb, 11, s.stride, s.pad, out_layout="NCHW")
    assert torch.equal(planar.cpu(), torch.from_numpy(oracle.unpack_nchwc(ref))), U.last_variant()
    del planar, ref
    q_ref = oracle.conv2d_nchwc_u8_requant(data, wt, bias, 3, 16, s.stride, s.pad, 1, conv=oracle.c_conv2d_nchwc)
    q = U.conv2d_NCHWc_int8_requant(_t(data, dev), wp, tb, 3, 16, s.stride, s.pad)
    assert torch.equal(q.cpu(), torch.from_numpy(q_ref)), U.last_variant()


REL_TOL = 1e-2  # the tolerance BASELINE states for fp16 (max relative error against float64 on the fp16-rounded inputs)


def _max_rel(got, ref):
    return float((np.abs(got - ref) / np.maximum(np.abs(ref), 1e-3 * np.abs(ref).max())).max())


@pytest.mark.parametrize("s", [s for s in WL.RESNET50 if s.C % 16 == 0], ids=lambda s: s.name)
def test_resnet50_batch32_layer_fp16(dev, oracle, s):
    """fp16 variant of the sweep: valid convolution on the pre-padded input (the operator has no padding argument,
    python/tensorizer/ops/gpu.py:8-53), reference layout and prepared weights, against float64."""
    hp, wp = s.H + 2 * s.pad, s.W + 2 * s.pad
    a = rng.normal_f16((32, s.C // 16, hp, wp, 16), 9500 + s.C + s.K)
    b = rng.normal_f16((s.K // 16, s.C // 16, s.KH, s.KW, 16, 16), 9600 + s.K, 1.0 / np.sqrt(s.C * s.KH * s.KW))
    ref = oracle.conv2d_nchw16c_f16(a, b, s.stride, s.stride)
    ta, tb = _t(a, dev), _t(b, dev)
    out = U.conv2d_NCHW16c_OHWI16o(ta, tb, s.stride, s.stride, "float32")
    assert tuple(out.shape) == ref.shape
    assert _max_rel(out.cpu().numpy(), ref) <= REL_TOL, U.last_variant()
    prepared = U.conv2d_NCHW16c_OHWI16o(ta, U.prepare_conv2d_weight(tb), s.stride, s.stride, "float32")
    assert _max_rel(prepared.cpu().numpy(), ref) <= REL_TOL, U.last_variant()


def test_int8_gemm_4096_cubed_bit_exact(dev, oracle):
    """BASELINE config 1 at full size against the VNNI oracle: un-packed and pre-packed weights, every element."""
    M = N = K = 4096
    a = rng.uniform_u8((M, K), 9701)
    w = rng.uniform_s8((N, K), 9702)
    wp = oracle.prepack_dense_weight(w)
    ref = torch.from_numpy(oracle.c_dense(a, wp))
    ta = _t(a, dev)
    assert torch.equal(U.dense(ta, _t(w, dev)).cpu(), ref), U.last_variant()
    assert torch.equal(U.dense_dotprod(ta, _t(wp, dev)).cpu(), ref), U.last_variant()


def _random_mid_cases(count, seed):
    r = np.random.RandomState(seed)
    cases = []
    for _ in range(count):
        ks = int(r.choice([1, 1, 3]))
        cases.append((int(r.choice([1, 2, 4, 8, 16])), 16 * int(r.randint(1, 33)), int(r.randint(7, 41)), int(r.randint(7, 41)),
                      16 * int(r.randint(1, 33)), ks, int(r.choice([1, 1, 2])), ks // 2))
    return cases


@pytest.mark.parametrize("case", _random_mid_cases(24, 20250101), ids=lambda c: "x".join(str(v) for v in c))
def test_heuristic_choices_on_random_mid_size_layers(dev, oracle, monkeypatch, case):
    """Shapes outside the tuned tables (the tables are switched off): whatever variant the heuristic picks, the int8
    result is bit-exact on both weight layouts and the fp16 one within tolerance."""
    monkeypatch.setenv("UNIT_AMD_CONV_NOTABLE", "1")
    n, c, h, w, k, ks, stride, pad = case
    data = rng.uniform_u8((n, c // 16, h, w, 16), 9800 + c)
    wt = rng.uniform_s8((k // 16, c // 16, ks, ks, 4, 16, 4), 9801 + k)
    ref = oracle.c_conv2d_nchwc(data, wt, stride, pad, 1)
    td, tw = _t(data, dev), _t(wt, dev)
    assert np.array_equal(U.conv2d_NCHWc_int8(td, tw, stride, pad).cpu().numpy(), ref), U.last_variant()
    out = U.conv2d_NCHWc_int8(td, U.prepare_conv2d_weight(tw), stride, pad)
    assert np.array_equal(out.cpu().numpy(), ref), U.last_variant()
    if n <= 4:  # the float64 oracle is numpy
        hp, wp = h + 2 * pad, w + 2 * pad
        a = rng.normal_f16((n, c // 16, hp, wp, 16), 9802 + c)
        b = rng.normal_f16((k // 16, c // 16, ks, ks, 16, 16), 9803 + k, 1.0 / np.sqrt(c * ks * ks))
        fref = oracle.conv2d_nchw16c_f16(a, b, stride, stride)
        got = U.conv2d_NCHW16c_OHWI16o(_t(a, dev), U.prepare_conv2d_weight(_t(b, dev)), stride, stride, "float32")
        assert _max_rel(got.cpu().numpy(), fref) <= REL_TOL, U.last_variant()
