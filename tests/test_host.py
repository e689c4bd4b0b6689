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
                kinds = (1, 2) if path.endswith("_prepared.inc") else (1,)
                assert L.unit_conv_variant_is_direct(variant) in kinds, (path, row)


def test_registry_keeps_the_reference_fragment_keys():
    # python/tensorizer/intrinsics/intrinsics.py:28-39
    for key in ("tensorcore.load_a", "tensorcore.load_b", "tensorcore.store_c"):
        assert U.INTRINSICS[key]["part_of"] is U.INTRINSICS["mfma.f16"]


def test_bench_final_line_fits_the_tail_budget():
    """The driver keeps a tail of a few KiB of stdout: the last line must be one complete JSON object under 2 KiB
    even with every field at a plausible maximum width."""
    import json

    import bench
    line = {
        "metric": "int8 conv2d TOPS & % int8 MFMA peak (ResNet-50 b32); fp16 GEMM TFLOPS", "value": 123456.78,
        "unit": "TOP/s", "n_gpus": 1, "steps": 1000, "warmup": 100, "ms_per_step": 1234.5678, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "ResNet-50 v1 conv stack (53 convs, 20 shapes), batch 32, int8 u8 x s8 -> i32, "
                               "NCHW16c / NCHW4c stem (BASELINE.json configs[4])",
                   "batch": 32, "ops_per_step": 246779215872, "weights": "prepared"},
        "pct_int8_mfma_peak": 99.99, "bit_exact_vs_oracle": True,
        "roofline": dict(bound="hbm", achieved=4412.8, peak=8000.0, unit="GB/s", frac=0.5516, frac_cold=0.5012,
                         traffic=115840483, traffic_source="profiles/conv_i8_resnet50_b32_1x1_64_256_56.txt",
                         kernel="i8prep_c16_x64_y64_g1_d2w4n_r2_s1", layer="1x1s2_1024_2048@14", launch_us=24.75,
                         launch_us_cold=26.11),
        "cpu_baseline": dict(value=5.634, unit="TOP/s", cores=16, kind="port", vnni=True,
                             sample="same step by the AVX-512 VNNI oracle: 20 unique layers, warm-up + repeat=10 x "
                                    "number=3 each, mean x multiplicity",
                             seconds=0.044, gemm_int8_tops=17.61, gemm_fp16_tflops=1.31),
        "best_mfma_bound_layer": dict(layer="3x3_512_512@7", us=9.67, pct_int8_peak=15.2),
        "gemm_int8_us": 80.39, "gemm_int8_pct_peak": 33.97, "gemm_int8_prepared_w_us": 72.31, "gemm_int8_prepared_w_pct_peak": 37.77, "gemm_fp16_us": 143.58, "gemm_fp16_tflops": 957.2,
        "gemm_fp16_pct_peak": 38.05, "gemm_fp16_prepared_b_us": 119.64, "gemm_fp16_prepared_b_pct_peak": 45.66,
        "gemm_fp16_max_rel_err": 0.000247, "sum_layers_cold_us": 612.3, "launch": "hipgraph",
        "roofline_step": dict(ideal_us=217.2, frac=0.377, bytes=1702945984, ops=246779215872, launches=53),
        "fp16_conv": dict(stack_us=618.2, tflops=387.0),
        "gemm_int8_frac_of_probe": 0.565, "gemm_fp16_frac_of_probe": 0.737,
        "probe": {"int8_tops": 4409.7, "fp16_tflops": 2327.2, "int8_tops_bench_operands": 3374.3,
                  "fp16_tflops_bench_operands": 1646.7},
    }
    s = bench.compact_line(dict(line))
    assert len(s) <= bench.FINAL_LINE_BUDGET and "\n" not in s
    back = json.loads(s)
    for key in ("metric", "value", "unit", "ms_per_step", "roofline", "roofline_step", "cpu_baseline", "config",
                "gemm_int8_frac_of_probe", "gemm_fp16_frac_of_probe"):
        assert key in back
    # an oversized line sheds optional keys, never the contract's
    line["probe"] = {f"k{i}": "x" * 40 for i in range(40)}
    back = json.loads(bench.compact_line(dict(line)))
    assert "probe" not in back and "roofline" in back and "cpu_baseline" in back


def test_bench_traffic_table_names_its_profiles():
    import os
    import re

    import bench
    table = bench.read_traffic_table()
    assert table, "profiles/hbm_traffic_table.txt is missing or empty"
    root = os.path.dirname(bench.__file__)
    tuned = open(os.path.join(root, "unit_amd", "csrc", "tuned_conv_i8_prepared.inc")).read()
    for (layer, kernel), (nbytes, src) in table.items():
        assert any(s.name == layer for s in WL.RESNET50) and nbytes > 0
        assert os.path.exists(os.path.join(root, src)), src
        # the row describes the kernel variant that the tuned table picks for this layer at batch 32 (the benchmark's
        # launch), and the profile it points to was taken on that variant: otherwise bench.py would report no traffic
        m = re.search(r"resnet50 b32 " + re.escape(layer) + r": [0-9.]+ us \(([^)]*)\)", tuned)
        assert m and m.group(1) == kernel, (layer, kernel, m and m.group(1))
        assert f"unit_last_variant(): {kernel}" in open(os.path.join(root, src)).read(), src


def test_padding_bound_is_checked_on_the_host():
    import ctypes

    from unit_amd import _lib
    L = _lib.load()
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    ok = _lib.ConvDesc(1, 16, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 16)
    assert L.unit_conv_out_hw(ctypes.byref(ok), ctypes.byref(oh), ctypes.byref(ow)) == 0 and (oh.value, ow.value) == (8, 8)
    bad = _lib.ConvDesc(1, 16, 8, 8, 16, 3, 3, 1, 1, 16384, 1, 1, 1, 1, 1, 16)
    assert L.unit_conv_out_hw(ctypes.byref(bad), ctypes.byref(oh), ctypes.byref(ow)) != 0
    assert b"padding" in L.unit_last_error()
