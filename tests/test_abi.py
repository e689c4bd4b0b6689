"""The C-ABI library loads and exports every symbol include/unit_amd.h declares; argument
validation that needs no GPU (nothing here launches a kernel)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "unit_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(unit_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from unit_amd import _lib
    lib = _lib.load()
    names = header_functions()
    assert len(names) >= 16
    for n in names:
        assert hasattr(lib, n), f"libunit_amd.so does not export {n}"
    assert sorted(_lib.SYMBOLS) == names, "unit_amd/_lib.py and include/unit_amd.h disagree"
    assert lib.unit_version() == 106


def test_conv_desc_matches_the_header_struct():
    from unit_amd import _lib
    text = open(os.path.join(ROOT, "include", "unit_amd.h")).read()
    body = re.search(r"typedef struct unit_conv_desc \{(.*?)\} unit_conv_desc;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = [f.strip() for decl in re.findall(r"int32_t ([^;]+);", body) for f in decl.split(",")]
    assert fields == [f for f, _ in _lib.ConvDesc._fields_]
    assert ctypes.sizeof(_lib.ConvDesc) == 4 * len(fields)


def test_conv3d_desc_matches_the_header_struct():
    from unit_amd import _lib
    text = open(os.path.join(ROOT, "include", "unit_amd.h")).read()
    body = re.search(r"typedef struct unit_conv3d_desc \{(.*?)\} unit_conv3d_desc;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = [f.strip() for decl in re.findall(r"int32_t ([^;]+);", body) for f in decl.split(",")]
    assert fields == [f for f, _ in _lib.Conv3dDesc._fields_]


def test_out_hw_and_error_paths_without_gpu():
    from unit_amd import _lib
    L = _lib.load()
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    d = _lib.ConvDesc(1, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 16)
    assert L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)) == 0
    assert (oh.value, ow.value) == (56, 56)
    d = _lib.ConvDesc(1, 4, 224, 224, 64, 7, 7, 2, 2, 3, 3, 3, 3, 1, 1, 4)
    assert L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)) == 0
    assert (oh.value, ow.value) == (112, 112)
    d = _lib.ConvDesc(1, 16, 4, 4, 16, 5, 5, 1, 1, 0, 0, 0, 0, 1, 1, 16)
    assert L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)) == -1
    assert b"window" in L.unit_last_error()
    # null pointers and bad shapes are rejected before anything touches a device
    assert L.unit_dense_u8s8s32(None, None, None, 4, 4, 16, None) == -1
    assert L.unit_dense_dotprod_u8s8s32(1, 1, 1, 4, 100, 16, None) == -1 and b"multiple of 128" in L.unit_last_error()
    assert L.unit_dense_u8s8s32(1, 1, 1, 4, 4, 10, None) == -1 and b"multiple of 16" in L.unit_last_error()
    assert L.unit_gemm_f16(1, 1, 1, 4, 4, 5, 0, None) == -1
    assert L.unit_pack_nchwc(1, 1, 1, 3, 4, 4, 4, 3, None) == -1 and b"elem_size" in L.unit_last_error()
    assert L.unit_prepack_conv_weight_s8(1, 1, 16, 16, 3, 3, 8, None) == -1
    bad = _lib.ConvDesc(1, 24, 8, 8, 16, 3, 3, 1, 1, 0, 0, 0, 0, 1, 1, 16)  # C % cb != 0
    assert L.unit_conv2d_nchwc_u8s8s32(ctypes.byref(bad), 1, 1, 1, None) == -1
    pad = _lib.ConvDesc(1, 16, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 16)  # fp16 op has no padding argument
    assert L.unit_conv2d_nchw16c_f16f32(ctypes.byref(pad), 1, 1, 1, None) == -1
    # the fused signed form and the 3-D operator validate the same way
    assert L.unit_conv2d_nchwc_s8s8s32_fused(ctypes.byref(bad), 1, 1, None, 11, 1, None) == -1
    assert L.unit_conv2d_nchwc_s8s8s32_fused(None, 1, 1, None, 11, 1, None) == -1 and b"null" in L.unit_last_error()
    d3 = _lib.Conv3dDesc(1, 18, 16, 8, 8, 16, 3, 3, 3, 1)  # C % 4 != 0
    assert L.unit_conv3d_ncdhwc_s8s8s32(ctypes.byref(d3), 1, 1, 1, None) == -1 and b"multiple of 4" in L.unit_last_error()
    d3 = _lib.Conv3dDesc(1, 4, 16, 20, 20, 16, 3, 3, 9, 1)  # 4-channel blocks: rows of at most 8 taps
    assert L.unit_conv3d_ncdhwc_s8s8s32(ctypes.byref(d3), 1, 1, 1, None) == -1 and b"KW <= 8" in L.unit_last_error()
    d3 = _lib.Conv3dDesc(1, 16, 2, 8, 8, 16, 3, 3, 3, 1)   # kernel deeper than the input
    assert L.unit_conv3d_ncdhwc_s8s8s32(ctypes.byref(d3), 1, 1, 1, None) == -1 and b"window" in L.unit_last_error()
    assert L.unit_conv_variant_count() >= 70
    kinds = [L.unit_conv_variant_is_direct(v) for v in range(L.unit_conv_variant_count())]
    assert set(kinds) == {0, 1, 2} and kinds.count(1) >= 20 and kinds.count(2) >= 4
    assert L.unit_conv_variant_is_direct(-1) == -1 and L.unit_conv_variant_is_direct(len(kinds)) == -1
    # prepared weights: size formula ceil(K/32) * k-steps * 1 KiB (+ 128 bytes of addends per block and 16 KiB of
    # zeros, the lines the LDS-shared kernels fetch for padded taps, for int8)
    nb = ctypes.c_size_t()
    assert L.unit_conv2d_prepared_weight_bytes(256, 256, 3, 3, 16, 1, ctypes.byref(nb)) == 0 and nb.value == 8 * 72 * 1024 + 8 * 128 + 16384
    assert L.unit_conv2d_prepared_weight_bytes(48, 16, 3, 3, 16, 1, ctypes.byref(nb)) == 0 and nb.value == 2 * 5 * 1024 + 2 * 128 + 16384
    assert L.unit_conv2d_prepared_weight_bytes(48, 16, 3, 3, 16, 2, ctypes.byref(nb)) == 0 and nb.value == 2 * 9 * 1024
    # 4-channel blocks: one k-step per (channel block, kh)
    assert L.unit_conv2d_prepared_weight_bytes(64, 4, 7, 7, 4, 1, ctypes.byref(nb)) == 0 and nb.value == 2 * 7 * 1024 + 2 * 128 + 16384
    assert L.unit_conv2d_prepared_weight_bytes(64, 4, 9, 9, 4, 1, ctypes.byref(nb)) == -1 and b"KW <= 8" in L.unit_last_error()
    assert L.unit_conv2d_prepared_weight_bytes(64, 4, 3, 3, 4, 2, ctypes.byref(nb)) == -1 and b"cb must be" in L.unit_last_error()
    assert L.unit_conv2d_prepared_weight_bytes(40, 16, 3, 3, 16, 1, ctypes.byref(nb)) == -1 and b"multiple of 16" in L.unit_last_error()
    assert L.unit_conv2d_prepared_weight_bytes(48, 16, 3, 3, 16, 4, ctypes.byref(nb)) == -1 and b"elem_bytes" in L.unit_last_error()
    assert L.unit_conv2d_prepare_weight(48, 16, 3, 3, 16, 1, None, 1, None) == -1 and b"null" in L.unit_last_error()
    c4 = _lib.ConvDesc(1, 4, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 2, 4)
    assert L.unit_conv2d_nchwc_u8s8s32_prepared(ctypes.byref(c4), 1, 1, 1, None) == -1 and b"dilation along W" in L.unit_last_error()
    c8 = _lib.ConvDesc(1, 8, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 8)
    assert L.unit_conv2d_nchwc_u8s8s32_prepared(ctypes.byref(c8), 1, 1, 1, None) == -1 and b"cb must be" in L.unit_last_error()
    big = _lib.ConvDesc(1, 16, 20, 20, 16, 7, 7, 1, 1, 0, 0, 0, 0, 1, 1, 16)
    assert L.unit_conv2d_nchwc_s8s8s32_fused_prepared(ctypes.byref(big), 1, 1, None, 1, 1, None) == -1 and b"31 positions" in L.unit_last_error()
    pad = _lib.ConvDesc(1, 16, 20, 20, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 16)
    assert L.unit_conv2d_nchw16c_f16f32_prepared(ctypes.byref(pad), 1, 1, 1, None) == -1 and b"padding" in L.unit_last_error()
    # NCHW output: the channel count must round up to K
    ok32 = _lib.ConvDesc(1, 16, 8, 8, 32, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 16)
    for oc in (16, 33, 0, -1):
        assert L.unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw(ctypes.byref(ok32), 16, 16, None, 1, 16, oc, None) == -1
        assert b"does not round up" in L.unit_last_error()
    assert L.unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw(ctypes.byref(ok32), 16, 16, None, 1, 8, 17, None) == -1
    assert b"aligned" in L.unit_last_error()
    assert L.unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw(None, 16, 16, None, 1, 16, 17, None) == -1 and b"null" in L.unit_last_error()
    # tensor pointers must be 16-byte aligned (the kernels use 16-byte vector accesses)
    ok = _lib.ConvDesc(1, 16, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 16)
    for args in ((8, 16, 16), (16, 4, 16), (16, 16, 24)):
        assert L.unit_conv2d_nchwc_u8s8s32(ctypes.byref(ok), *args, None) == -1 and b"aligned" in L.unit_last_error()
        assert L.unit_conv2d_nchwc_u8s8s32_prepared(ctypes.byref(ok), *args, None) == -1 and b"aligned" in L.unit_last_error()
    assert L.unit_dense_u8s8s32(16, 16, 8, 16, 16, 16, None) == -1 and b"aligned" in L.unit_last_error()
    assert L.unit_gemm_f16(16, 2, 16, 16, 16, 16, 0, None) == -1 and b"aligned" in L.unit_last_error()
    # fp16 GEMM on a prepared b
    assert L.unit_gemm_f16_prepare_b(16, 16, 12, 16, None) == -1 and b"multiple of 8" in L.unit_last_error()
    assert L.unit_gemm_f16_prepare_b_packed32(16, 16, 48, 64, None) == -1 and b"multiples of 32" in L.unit_last_error()
    assert L.unit_gemm_f16_prepare_b_packed32(16, None, 64, 64, None) == -1 and b"null" in L.unit_last_error()
    assert L.unit_gemm_f16_prepare_b_packed32(16, 8, 64, 64, None) == -1 and b"aligned" in L.unit_last_error()
    assert L.unit_gemm_f16_prepared(16, 16, 16, 16, 6, 16, 0, None) == -1 and b"multiple of 4" in L.unit_last_error()
    assert L.unit_gemm_f16_prepared(16, None, 16, 16, 8, 16, 0, None) == -1 and b"null" in L.unit_last_error()
    assert L.unit_gemm_f16_prepared(16, 8, 16, 16, 8, 16, 0, None) == -1 and b"aligned" in L.unit_last_error()
    # size limit: weights, GEMM operands and a single image of a convolution stay below 2^31 bytes (32-bit
    # offsets in the kernels); a larger batch is sliced instead and reaches the pointer checks
    huge = _lib.ConvDesc(2, 256, 4096, 4096, 256, 1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 16)
    many = _lib.ConvDesc(4096, 256, 56, 56, 256, 1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 16)
    assert L.unit_conv2d_nchwc_u8s8s32(ctypes.byref(many), 1, 1, 1, None) == -1 and b"aligned" in L.unit_last_error()
    assert L.unit_conv2d_nchwc_u8s8s32(ctypes.byref(huge), 1, 1, 1, None) == -1 and b"2^31" in L.unit_last_error()
    assert L.unit_dense_u8s8s32(1, 1, 1, 16, 65536, 65536, None) == -1 and b"2^31" in L.unit_last_error()
    assert L.unit_dense_u8s8s32(1, 1, 1, 65536, 65536, 16, None) == -1 and b"aligned" in L.unit_last_error()  # row slices
    with pytest.raises(ValueError):
        _lib.check(-1)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from unit_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.UnitError, match="no CPU fallback"):
        _lib.load()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "unit_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")) or f == "Makefile":
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"
