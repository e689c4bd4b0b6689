"""Host-side logic of the operator entry points (no GPU): argument checks, registry, workloads."""
import numpy as np
import pytest
import torch

import unit_amd as U
from unit_amd import workloads as WL


def test_ops_refuse_cpu_tensors_instead_of_falling_back():
    data = torch.zeros((1, 4, 8, 8, 16), dtype=torch.uint8)
    wt = torch.zeros((4, 4, 3, 3, 4, 16, 4), dtype=torch.int8)
    with pytest.raises(ValueError, match="GPU"):
        U.conv2d_NCHWc_int8(data, wt, 1, 1)
    with pytest.raises(ValueError, match="GPU"):
        U.dense_dotprod(torch.zeros((4, 16), dtype=torch.uint8), torch.zeros((1, 4, 128, 4), dtype=torch.int8))
    with pytest.raises(ValueError, match="GPU"):
        U.gemm_fp16(torch.zeros((4, 8), dtype=torch.float16), torch.zeros((8, 4), dtype=torch.float16))
    with pytest.raises(TypeError):
        U.conv2d_NCHWc_int8(np.zeros((1, 4, 8, 8, 16), np.uint8), wt, 1, 1)
    with pytest.raises(ValueError, match="GPU"):
        U.conv2d_NCHWc_int8_fused(data.view(torch.int8), wt, None, 11, 1, 1)
    with pytest.raises(ValueError, match="GPU"):
        U.conv3d_NCDHWc_int8(torch.zeros((1, 1, 4, 8, 8, 16), dtype=torch.int8),
                             torch.zeros((1, 1, 3, 3, 3, 4, 16, 4), dtype=torch.int8))


def test_conv_out_hw_matches_reference_shapes():
    # cpu-shapes.log:377 logs 58x58 for the padded 56x56 3x3 layer; :380 230x230 for the 224 stem
    assert U.conv_out_hw(56, 56, 3, 3, 1, 1) == (56, 56)
    assert U.conv_out_hw(58, 58, 3, 3, 1, 0) == (56, 56)
    assert U.conv_out_hw(224, 224, 7, 7, 2, 3) == (112, 112)
    assert U.conv_out_hw(230, 230, 7, 7, (2, 2), (0, 0, 0, 0)) == (112, 112)
    assert U.conv_out_hw(14, 14, 3, 3, 1, 2, 2) == (14, 14)
    with pytest.raises(ValueError):
        U.conv_out_hw(4, 4, 5, 5, 1, 0)


def test_registry_keeps_select_by_name():
    assert U.INTRINSICS["vnni"] is U.INTRINSICS["mfma.i8"]
    assert U.INTRINSICS["tensorcore"] is U.INTRINSICS["mfma.f16"]
    assert U.INTRINSICS["mfma.i8"]["conv2d"] is U.conv2d_NCHWc_int8
    assert U.INTRINSICS["mfma.i8"]["dense"] is U.dense_dotprod
    assert U.INTRINSICS["mfma.f16"]["pattern"]["tile"] == (32, 32, 16)


def test_workloads():
    assert len(WL.RESNET18) == 11 and len(WL.RESNET50) == 20
    assert sum(s.count for s in WL.RESNET50) == 53 and sum(s.count for s in WL.RESNET18) == 20
    s = WL.SINGLE_CONV
    assert WL.macs(s, 1) == 115605504  # 115.6 M MAC for the single-convolution benchmark configuration
    assert WL.algorithmic_bytes(s, 1) == 200704 + 36864 + 802816
    stem = WL.RESNET50[0]
    assert WL.channel_block(stem.C) == 4 and WL.channel_block(64) == 16
    assert WL.macs(stem, 1, logical=False) * 3 == WL.macs(stem, 1) * 4
    # ResNet-50 convolutions: ~3.86 G MAC per image
    total = sum(WL.macs(s, 1) * s.count for s in WL.RESNET50)
    assert 3.8e9 < total < 3.9e9


def test_rng_streams():
    from unit_amd import rng
    u = rng.uniform_u8((1 << 16,), 1)
    s = rng.uniform_s8((1 << 16,), 2)
    assert u.min() == 0 and u.max() == 255 and s.min() == -128 and s.max() == 127
    assert abs(float(u.mean()) - 127.5) < 1.5 and abs(float(s.astype(np.float64).mean())) < 1.5
    z = rng.normal_f16((1 << 16,), 3).astype(np.float64)
    assert abs(z.mean()) < 0.02 and abs(z.std() - 1.0) < 0.02
    assert np.array_equal(rng.uniform_u8((100,), 5), rng.uniform_u8((100,), 5))
    assert not np.array_equal(rng.uniform_u8((100,), 5), rng.uniform_u8((100,), 6))


def test_relay_driver_wants_ten_integers():
    from unit_amd import relay
    with pytest.raises(SystemExit, match="usage"):
        relay.main(["1", "2", "3"])
    with pytest.raises(SystemExit, match="differ"):
        relay.main("1 32 14 14 32 16 3 3 1 1".split())


def test_resnet50_chain_lists_the_logged_shapes():
    """The chain's 52 layers are exactly the reference's ResNet-50 shape list without the stem, with its multiplicities."""
    from collections import Counter
    from unit_amd import chain
    layers = chain.resnet50_layers(lambda oc, ic, k: (oc, ic, k))
    assert len(layers) == 52
    hw, seen = {-1: 56}, Counter()
    for i, ly in enumerate(layers):
        src = i - 1 if ly.source is None else ly.source
        assert -1 <= src < i
        oc, ic, k = ly.weight
        seen[(ic, hw[src], oc, k, ly.stride, ly.padding)] += 1
        hw[i] = (hw[src] + 2 * ly.padding - k) // ly.stride + 1
        if src >= 0:
            assert layers[src].weight[0] == ic  # reads as many channels as its source writes
    want = Counter({(s.C, s.H, s.K, s.KH, s.stride, s.pad): s.count for s in WL.RESNET50[1:]})
    assert seen == want


def test_resnet18_chain_lists_the_logged_shapes():
    from collections import Counter
    from unit_amd import chain
    layers = chain.resnet18_layers(lambda oc, ic, k: (oc, ic, k))
    assert len(layers) == 19
    hw, seen = {-1: 56}, Counter()
    for i, ly in enumerate(layers):
        assert -1 <= ly.source < i
        oc, ic, k = ly.weight
        seen[(ic, hw[ly.source], oc, k, ly.stride, ly.padding)] += 1
        hw[i] = (hw[ly.source] + 2 * ly.padding - k) // ly.stride + 1
        if ly.source >= 0:
            assert layers[ly.source].weight[0] == ic
    want = Counter({(s.C, s.H, s.K, s.KH, s.stride, s.pad): s.count for s in WL.RESNET18[1:]})
    assert seen == want


def test_tuned_tables_name_existing_variants():
    """Every row of the tuned tables compiled into the library names a kernel variant that exists; the tables for
    prepared weights only name direct variants (the only ones that read the prepared layout)."""
    import glob
    import os
    import re
    from unit_amd import _lib
    L = _lib.load()
    count = L.unit_conv_variant_count()
    csrc = os.path.join(os.path.dirname(os.path.abspath(U.__file__)), "csrc")
    files = sorted(glob.glob(os.path.join(csrc, "tuned_conv_*.inc")))
    assert len(files) == 4
    for path in files:
        rows = re.findall(r"\{([^}]*)\}", open(path).read())
        assert rows, path
        keys = set()
        for row in rows:
            npix, k, c, kh, kw, sh, variant, splits, panel = (int(v) for v in row.split(","))
            assert 0 <= variant < count and splits >= 1 and panel >= 0, (path, row)
            assert (npix, k, c, kh, kw, sh) not in keys, (path, row)  # one choice per shape
            keys.add((npix, k, c, kh, kw, sh))
            if path.endswith("_prepared.inc"):
                assert L.unit_conv_variant_is_direct(variant) == 1, (path, row)
