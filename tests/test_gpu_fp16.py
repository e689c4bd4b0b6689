"""Parity of the fp16 HIP path against a float64 reference on the fp16-rounded inputs.
Tolerance of the fp16 path: max |d| / max(|ref|, eps * max|ref|) <= 1e-2."""
import numpy as np
import pytest
import torch

import unit_amd as U
from unit_amd import rng

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def max_rel(out, ref):
    ref = np.asarray(ref, dtype=np.float64)
    floor = 1e-3 * np.abs(ref).max()
    return float((np.abs(out.astype(np.float64) - ref) / np.maximum(np.abs(ref), floor)).max())


def test_mfma_tile_f16_lane_layout(dev):
    import ctypes
    from unit_amd import _lib
    a = (rng.uniform_s8((32, 16), 1) % 5).astype(np.float16)
    b = (rng.uniform_s8((32, 16), 2) % 7).astype(np.float16)
    ta, tb = _t(a, dev), _t(b, dev)
    tc = torch.zeros((32, 32), dtype=torch.float32, device=dev)
    _lib.check(_lib.load().unit_mfma_tile_f16(ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), None))
    torch.cuda.synchronize()
    assert np.array_equal(tc.cpu().numpy(), (a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))


GEMM_CASES = [(128, 768, 3072), (32, 32, 64), (100, 132, 72), (512, 4096, 256), (4096, 2048, 512), (2050, 4100, 136),
              (1024, 4096, 128), (300, 264, 96),     # both operands straight into LDS, 128 x 128 tiles, whole and ragged
              (2050, 4104, 192), (2050, 4104, 160),  # the same on 256 x 256 tiles, 128- and 64-byte stages, ragged
              (1000, 4100, 192), (2050, 4100, 192),  # N not a multiple of 8: b through the transposing register loader
              (1, 8, 64), (3, 16, 96), (260, 8, 128)]  # one row, one 8-column chunk, one stage


@pytest.mark.parametrize("M,N,K", GEMM_CASES)
@pytest.mark.parametrize("out_dtype", ["float32", "float16"])
def test_gemm_fp16(dev, oracle, M, N, K, out_dtype):
    a = rng.normal_f16((M, K), 31 + M, 1.0 / np.sqrt(K))
    b = rng.normal_f16((K, N), 57 + N)
    out = U.gemm_fp16(_t(a, dev), _t(b, dev), out_dtype)
    torch.cuda.synchronize()
    ref = oracle.gemm_f16(a, b)
    err = max_rel(out.cpu().numpy(), ref)
    assert err <= (REL_TOL if out_dtype == "float32" else REL_TOL), (err, U.last_variant())


@pytest.mark.parametrize("M,N,K", [(128, 768, 3072), (96, 200, 2056), (1, 8, 4096), (300, 260, 520)])
def test_gemm_fp16_k_splits(dev, oracle, M, N, K):
    """Few output tiles, long reduction (apps/gpu/gemm.py:6 is 128 x 768 x 3072): the reduction is shared between
    workgroups that add into the zero-filled fp32 output; fp16 output keeps one workgroup per tile."""
    a = rng.normal_f16((M, K), 131 + M, 1.0 / np.sqrt(K))
    b = rng.normal_f16((K, N), 157 + N)
    ta, tb = _t(a, dev), _t(b, dev)
    ref = oracle.gemm_f16(a, b)
    for operand in (tb, U.prepare_gemm_b(tb)):
        out = U.gemm_fp16(ta, operand)
        torch.cuda.synchronize()
        assert int(U.last_variant().rsplit("_s", 1)[1]) > 1, U.last_variant()
        assert max_rel(out.cpu().numpy(), ref) <= REL_TOL, U.last_variant()
        half = U.gemm_fp16(ta, operand, "float16")
        assert U.last_variant().endswith("_s1") and max_rel(half.cpu().numpy(), ref) <= REL_TOL


def test_gemm_fp16_k_splits_switched_off(dev, oracle, monkeypatch):
    """UNIT_AMD_GEMM_F16_SPLITK=1 keeps one workgroup per output tile: no fp32 atomics, so two runs give the same bits."""
    M, N, K = 128, 768, 3072
    a = rng.normal_f16((M, K), 141, 1.0 / np.sqrt(K))
    b = rng.normal_f16((K, N), 142)
    ta, tb = _t(a, dev), _t(b, dev)
    ref = oracle.gemm_f16(a, b)
    for operand in (tb, U.prepare_gemm_b(tb)):
        split = U.gemm_fp16(ta, operand)
        assert int(U.last_variant().rsplit("_s", 1)[1]) > 1, U.last_variant()
        monkeypatch.setenv("UNIT_AMD_GEMM_F16_SPLITK", "1")
        one = U.gemm_fp16(ta, operand)
        assert U.last_variant().endswith("_s1"), U.last_variant()
        again = U.gemm_fp16(ta, operand)
        monkeypatch.delenv("UNIT_AMD_GEMM_F16_SPLITK")
        assert torch.equal(one, again)
        assert max_rel(one.cpu().numpy(), ref) <= REL_TOL and max_rel(split.cpu().numpy(), ref) <= REL_TOL


PREPARED_GEMM_CASES = GEMM_CASES + [(4096, 4096, 1024), (2304, 2560, 192), (257, 260, 64), (3000, 2052, 200),
                                    (2048, 2048, 320)]  # 256 x 128 tiles: a direct to LDS, prepared b through registers


@pytest.mark.parametrize("M,N,K", PREPARED_GEMM_CASES)
@pytest.mark.parametrize("out_dtype", ["float32", "float16"])
def test_gemm_fp16_prepared_b(dev, oracle, M, N, K, out_dtype):
    """b re-laid once as (N, K): the transposed buffer is exact, the product is within tolerance of float64 and
    agrees with the plain entry to rounding (both sum k in ascending order of 16-element MFMA steps)."""
    a = rng.normal_f16((M, K), 31 + M, 1.0 / np.sqrt(K))
    b = rng.normal_f16((K, N), 57 + N)
    ta, tb = _t(a, dev), _t(b, dev)
    pb = U.prepare_gemm_b(tb)
    torch.cuda.synchronize()
    assert np.array_equal(pb.bt.cpu().numpy(), b.T)
    out = U.gemm_fp16(ta, pb, out_dtype)
    torch.cuda.synchronize()
    assert U.last_variant().startswith("f16gemmbt")
    ref = oracle.gemm_f16(a, b)
    err = max_rel(out.cpu().numpy(), ref)
    assert err <= REL_TOL, (err, U.last_variant())
    plain = U.gemm_fp16(ta, tb, out_dtype)
    assert max_rel(out.cpu().numpy(), plain.cpu().numpy().astype(np.float64)) <= 1e-3, U.last_variant()


def test_gemm_fp16_prepared_b_integer_exact(dev, oracle):
    M, N, K = 512, 768, 1024
    a = (np.arange(M * K).reshape(M, K) % 7).astype(np.float16)
    b = (np.arange(K * N).reshape(K, N) % 5 - 2).astype(np.float16)
    # 128 x 128 tiles with both operands straight into LDS, in two k-splits and whole; 256 x 256 tiles; and, with a
    # reduction that is no whole number of 64-byte stages, the register pipeline
    for (m, n, k), kernel in (((M, N, K), "dma_x128_y128_k64_w2x2_r4_s2"), ((4096, 2048, K), "dma_x128_y128_k64_w2x2_r4_s1"),
                              ((4096, 4096, K), "dma_x256_y256"), ((M, N, 1000), "f16gemmbt_x")):
        aa = np.resize(a, (m, k)); bb = np.resize(b, (k, n))
        out = U.gemm_fp16(_t(aa, dev), U.prepare_gemm_b(_t(bb, dev))).cpu().numpy()
        assert np.array_equal(out.astype(np.float64), oracle.gemm_f16(aa, bb)), U.last_variant()
        assert kernel in U.last_variant(), U.last_variant()


@pytest.mark.parametrize("M,N,K", [(64, 192, 1024), (128, 768, 3072), (300, 2080, 96), (4096, 4096, 512)])
def test_gemm_fp16_reference_packed_b(dev, oracle, M, N, K):
    """b handed over as the reference packs it, (N/32, K/32, 32, 32) (apps/gpu/gemm-pack.py:9,17; its own size is
    64 x 192 x 1024): prepared once and passed straight to gemm_fp16, against the oracle's packed GEMM; with
    integer-valued operands the result is exact and the re-laid operand equals b transposed."""
    a = rng.normal_f16((M, K), 6100 + M)
    b = rng.normal_f16((K, N), 6200 + N, 1.0 / np.sqrt(K))
    bp = oracle.pack_gemm_b32(b)
    tbp = _t(bp, dev)
    prepared = U.prepare_gemm_b(tbp)
    assert U.last_variant() == "f16_unpack32_b"
    assert np.array_equal(prepared.bt.cpu().numpy(), b.T)
    ref = oracle.gemm_f16_packed(a, bp) if M * N * K <= 1 << 28 else oracle.gemm_f16(a, b)
    for out in (U.gemm_fp16(_t(a, dev), prepared), U.gemm_fp16(_t(a, dev), tbp)):
        assert max_rel(out.cpu().numpy(), ref) <= REL_TOL, U.last_variant()
    ai = (np.arange(M * K).reshape(M, K) % 7).astype(np.float16)
    bi = (np.arange(K * N).reshape(K, N) % 5 - 2).astype(np.float16)
    out = U.gemm_fp16(_t(ai, dev), _t(oracle.pack_gemm_b32(bi), dev)).cpu().numpy()
    assert np.array_equal(out.astype(np.float64), oracle.gemm_f16(ai, bi)), U.last_variant()


def test_gemm_fp16_integer_exact(dev, oracle):
    """Small-integer operands (the arange % 7 recipe of apps/gpu/conv-wdim.py:33-36) make every
    fp32 partial sum exact, so the result must match the float64 reference bit for bit."""
    M, N, K = 256, 384, 512
    a = (np.arange(M * K).reshape(M, K) % 7).astype(np.float16)
    b = (np.arange(K * N).reshape(K, N) % 5 - 2).astype(np.float16)
    # b read back from LDS with the transposing read, on 128 x 128 tiles (k-splits and whole) and 256 x 256 tiles; N not
    # a multiple of 8: b transposed in registers; K no whole number of stages: both operands through registers
    for (m, n, k), kernel in (((M, N, K), "dmatr_x128_y128_k64_w2x2_r4_s4"), ((4096, 2048, K), "dmatr_x128_y128_k64_w2x2_r4_s1"),
                              ((4096, 4096, K), "dmatr_x256_y256_k128"), ((4096, 4096, 96), "dmatr_x256_y256_k64"),
                              ((2048, 2052, K), "hybrid_x256"), ((M, N, 1000), "f16gemm_x")):
        aa = np.resize(a, (m, k)); bb = np.resize(b, (k, n))
        out = U.gemm_fp16(_t(aa, dev), _t(bb, dev)).cpu().numpy()
        assert np.array_equal(out.astype(np.float64), oracle.gemm_f16(aa, bb)), U.last_variant()
        assert kernel in U.last_variant(), U.last_variant()


CONV_CASES = [
    # N, C, H, W, K, kernel, stride
    (1, 64, 16, 18, 64, 3, 1),     # apps/gpu/conv-wdim.py shape family
    (1, 16, 9, 9, 16, 1, 1),
    (2, 32, 12, 10, 48, 3, 2),
    (1, 256, 30, 30, 256, 3, 2),   # gpu-tune.log:27-28
    (1, 256, 56, 56, 128, 1, 1),   # gpu-tune.log:5-6
    (4, 128, 30, 30, 128, 3, 1),
    (32, 256, 16, 16, 256, 3, 1),  # batch 32, 256-channel tile
]


@pytest.mark.parametrize("N,C,H,W,K,ks,stride", CONV_CASES)
def test_conv2d_fp16(dev, oracle, N, C, H, W, K, ks, stride):
    a = rng.normal_f16((N, C // 16, H, W, 16), 5 + C)
    b = rng.normal_f16((K // 16, C // 16, ks, ks, 16, 16), 9 + K, 1.0 / np.sqrt(C * ks * ks))
    out = U.conv2d_NCHW16c_OHWI16o(_t(a, dev), _t(b, dev), stride, stride, "float32")
    torch.cuda.synchronize()
    ref = oracle.conv2d_nchw16c_f16(a, b, stride, stride)
    assert tuple(out.shape) == ref.shape
    err = max_rel(out.cpu().numpy(), ref)
    assert err <= REL_TOL, (err, U.last_variant())


@pytest.mark.parametrize("N,C,H,W,K,ks,stride", [(2, 80, 9, 11, 96, 3, 1), (1, 32, 5, 5, 16, 1, 1), (3, 256, 9, 9, 160, 3, 2)])
def test_conv2d_fp16_every_variant(dev, oracle, monkeypatch, N, C, H, W, K, ks, stride):
    """Every tile variant gives the same result; integer-valued data makes fp32 accumulation exact
    in any summation order, so the comparison with the float64 reference is bit for bit."""
    from unit_amd import _lib
    a = (rng.uniform_u8((N, C // 16, H, W, 16), 3 + C) % 7).astype(np.float16) - 3
    b = (rng.uniform_u8((K // 16, C // 16, ks, ks, 16, 16), 4 + K) % 5).astype(np.float16) - 2
    ref = oracle.conv2d_nchw16c_f16(a, b, stride, stride)
    ta, tb = _t(a, dev), _t(b, dev)
    count = _lib.load().unit_conv_variant_count()
    ran = set()
    for v in range(1, count + 1):
        if _lib.load().unit_conv_variant_is_direct(v - 1) == 2:
            continue  # LDS-shared variants exist for prepared weights only: the id runs the heuristic's choice here
        monkeypatch.setenv("UNIT_AMD_CONV_VARIANT", str(v))
        try:
            out = U.conv2d_NCHW16c_OHWI16o(ta, tb, stride, stride, "float32")
        except ValueError as e:  # a variant may only be refused for its LDS budget or its layout
            assert "LDS" in str(e) or "not available" in str(e), (v, str(e))
            continue
        torch.cuda.synchronize()
        ran.add((v, U.last_variant()))
        assert np.array_equal(out.cpu().numpy().astype(np.float64), ref), (v, U.last_variant())
    assert len({name for _, name in ran}) == len({v for v, _ in ran}) >= 46


def test_conv2d_fp16_unpacked_operands(dev, oracle):
    """4-D NCHW + OIHW operands are packed in-op like python/tensorizer/ops/gpu.py:25-33; integer
    data makes the comparison exact."""
    N, C, H, W, K = 1, 32, 10, 10, 32
    a = (np.arange(N * C * H * W).reshape(N, C, H, W) % 7).astype(np.float16)
    b = (np.arange(K * C * 9).reshape(K, C, 3, 3) % 5 - 2).astype(np.float16)
    out = U.conv2d_NCHW16c_OHWI16o(_t(a, dev), _t(b, dev), 1, 1).cpu().numpy()
    ref = oracle.conv2d_nchw16c_f16(oracle.pack_nchwc(a, 16), oracle.prepack_conv_weight_f16(b), 1, 1)
    assert np.array_equal(out.astype(np.float64), ref)


def test_fp16_golden_fixtures(dev):
    import os
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    g = np.load(os.path.join(gold, "fp16_gemm_24x36x40.npz"))
    assert max_rel(U.gemm_fp16(_t(g["a"], dev), _t(g["b"], dev)).cpu().numpy(), g["out"]) <= REL_TOL
    g = np.load(os.path.join(gold, "fp16_conv_3x3_c32_k32.npz"))
    out = U.conv2d_NCHW16c_OHWI16o(_t(g["a"], dev), _t(g["b"], dev), 1, 1).cpu().numpy()
    assert max_rel(out, g["out"]) <= REL_TOL


def test_gemm_fp16_full_size(dev):
    """4096^3, every element, tolerance 1e-2 max relative error: rows sampled against numpy float64 on the host pin a
    float64 product computed on the device, and that product checks all 16.8 M results of b as it lies, of the prepared
    b and of fp16 output."""
    M = N = K = 4096
    a = rng.normal_f16((M, K), 61, 1.0 / 64)
    b = rng.normal_f16((K, N), 62)
    ta, tb = _t(a, dev), _t(b, dev)
    ref = ta.double() @ tb.double()
    rows = np.arange(0, M, 97)
    host = a[rows].astype(np.float64) @ b.astype(np.float64)
    assert np.abs(ref[rows].cpu().numpy() - host).max() <= 1e-9 * np.abs(host).max()
    floor = 1e-3 * float(ref.abs().max())
    for operand, dtype in ((tb, "float32"), (U.prepare_gemm_b(tb), "float32"), (tb, "float16")):
        out = U.gemm_fp16(ta, operand, dtype)
        err = float(((out.double() - ref).abs() / ref.abs().clamp_min(floor)).max())
        assert err <= REL_TOL, (err, U.last_variant())


@pytest.mark.parametrize("M,N,K", [(128, 768, 3072), (256, 512, 8192), (100, 260, 1024), (512, 512, 256), (96, 64, 4096)])
@pytest.mark.parametrize("out_dtype", ["float32", "float16"])
def test_gemm_fp16_k_splits_through_a_workspace(dev, oracle, M, N, K, out_dtype):
    """unit_gemm_f16_ws: partial tiles of the k-splits in planes of a workspace, added in split order.  Within the
    1e-2 tolerance of float64 (2e-3 more for the final fp16 rounding), bit-identical from run to run, available
    for fp16 output; a shape that needs no k-splits asks for no workspace and gives unit_gemm_f16's result."""
    a = rng.normal_f16((M, K), 11 + M, 1.0 / np.sqrt(K))
    b = rng.normal_f16((K, N), 12 + N)
    ta, tb = _t(a, dev), _t(b, dev)
    need = U.gemm_fp16_workspace_bytes(M, N, K)
    ws = torch.full((need + 64,), 0xAB, dtype=torch.uint8, device=dev)  # stale contents must not matter
    out1 = U.gemm_fp16(ta, tb, out_dtype, workspace=ws)
    name = U.last_variant()
    ws.fill_(0x5C)
    out2 = U.gemm_fp16(ta, tb, out_dtype, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(out1, out2), name
    assert ("planes" in name) == (need > 0), (name, need)
    ref = oracle.gemm_f16(a, b)
    err = max_rel(out1.float().cpu().numpy(), ref)
    assert err <= REL_TOL + (2e-3 if out_dtype == "float16" else 0), (err, name)
    if need == 0:
        assert torch.equal(out1, U.gemm_fp16(ta, tb, out_dtype)), name
    else:
        with pytest.raises(ValueError, match="workspace"):
            U.gemm_fp16(ta, tb, out_dtype, workspace=ws[:need - 16])


def test_gemm_fp16_workspace_integer_data_is_exact(dev, oracle):
    """Integer-valued data: every partial sum is exact in fp32, so the planes add up to the float64 result bit for bit."""
    M, N, K = 128, 768, 3072
    a = (rng.uniform_u8((M, K), 5) % 7).astype(np.float16) - 3
    b = (rng.uniform_u8((K, N), 6) % 5).astype(np.float16) - 2
    out = U.gemm_fp16(_t(a, dev), _t(b, dev), "float32", workspace=True)
    torch.cuda.synchronize()
    assert "planes" in U.last_variant()
    assert np.array_equal(out.cpu().numpy().astype(np.float64), oracle.gemm_f16(a, b))
